"""Same public names as the reference's src/enzyme_ad/jax/__init__.py:1-12,
plus the host-side pieces that replace JAX here (`vjp`, `ops`)."""
from .primitives import (
    cpp_call,
    ffi_call,
    hlo_call,
    enzyme_jax_ir,
    optimize_module,
    export,
    XLAPipeline,
    JaXPipeline,
    full_optimization_pass_pipeline,
    optimization_passes,
    DefaultJaXPipeline,
    DefaultCPPPipeline,
    parse_pass_pipeline,
    vjp,
    jvp,
)
from . import ops
