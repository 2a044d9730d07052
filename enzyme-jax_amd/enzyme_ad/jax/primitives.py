"""API surface of the reference's `enzyme_ad.jax` (src/enzyme_ad/jax/primitives.py)
over the MI355X kernels.

Kept from the reference: the pipeline configuration objects (`JaXPipeline`,
`XLAPipeline`, :81-115), the pass-pipeline string builders
(`optimization_passes`, `full_optimization_pass_pipeline`, :118-223), the
decorator `enzyme_jax_ir(argv, pipeline_options, jit_options, inner_jit)`
(:1528-1590) and the entry-point names `ffi_call`, `cpp_call`, `hlo_call`,
`optimize_module`, `export`.

Changed: the decorated function is written with the operators of
`enzyme_ad.jax.ops` and runs eagerly on HIP streams; `vjp` below plays the role
of `jax.vjp` through the reference's `enzyme_vjp` rule (:1381-1486): it returns
the primal result and a function from result cotangents to argument cotangents.
The MLIR pass pipeline named by `pipeline_options` selects nothing here - the
fused kernels implement the optimized graph directly - but the strings are
still built, parsed and carried so that code written for the reference runs.
"""
import re
from collections.abc import Callable, Sequence
from typing import Any

import torch

from . import ops

LANG_CPP, LANG_LLVM, LANG_MHLO = 0, 1, 2     # enzyme_call.Language (enzyme_call.cc)


class PipelineConfig:
    """primitives.py:56-78."""

    def xla_runtime(self):
        raise NotImplementedError()

    def pass_pipeline(self):
        raise NotImplementedError()

    def mlir_ad(self):
        raise NotImplementedError()

    def stablehlo_inject(self):
        raise NotImplementedError()

    def ad_level(self):
        raise NotImplementedError()

    def export_llvm(self):
        raise NotImplementedError()


class XLAPipeline(PipelineConfig):
    """primitives.py:81-98 (LLVM-level AD of XLA-CPU code; CPU only there)."""

    def __init__(self, name=None):
        self.exportname = name

    def xla_runtime(self):
        return False

    def pass_pipeline(self):
        return ""

    def mlir_ad(self):
        return False

    def stablehlo_inject(self):
        return False

    def export_llvm(self):
        return self.exportname


class JaXPipeline(PipelineConfig):
    """primitives.py:101-115."""

    def __init__(self, passes=""):
        self.passes = passes

    def pass_pipeline(self):
        return self.passes

    def mlir_ad(self):
        return True

    def stablehlo_inject(self):
        return True

    def ad_level(self):
        return self.passes.count("enzyme-wrap")


# Pattern-list placeholder: the reference obtains ~1000 rewrite-pattern names
# from its C++ pass-list generator (Integrations/c/EnzymeXLA.cpp:951-1104).
# The list itself has no meaning for fused kernels; its knobs are kept.
def _pattern_list(**kw):
    parts = ["emi_fused_llama<1>"]
    parts.append("max_constant_expansion<1>(%d)" % kw["max_constant_threshold"])
    for k in ("no_nan", "all_finite"):
        if kw[k]:
            parts.append("%s<1>" % k)
    parts.append("transpose_propagate_%s<1>" % kw["transpose_propagate"])
    parts.append("reshape_propagate_%s<1>" % kw["reshape_propagate"])
    return ";".join(p for p in parts if p.split("<")[0] not in set(kw["excluded_passes"]))


def optimization_passes(
    *,
    inline: bool = True,
    no_nan: bool = False,
    all_finite: bool = False,
    transpose_propagate: str = "up",
    reshape_propagate: str = "up",
    max_constant_threshold: int = 1024,
    enable_licm_optimization_passes: bool = True,
    loop_unswitch_threshold: int = 10,
    excluded_passes: list = [],
    enable_scatter_gather_optimization_passes: bool = True,
    enable_pad_optimization_passes: bool = True,
    enable_self_to_convolution_like_passes: bool = False,
    enable_structured_tensors_detection_passes: bool = False,
    enable_structured_tensors_passes: bool = True,
    enable_slice_to_batch_passes: bool = False,
    enable_reduce_slice_fusion_passes: bool = True,
    enable_concat_to_batch_passes: bool = True,
    enable_loop_raising_passes: bool = True,
    aggressive_propagation: bool = True,
):
    """Same keywords and string structure as primitives.py:118-192."""
    for name, val in (("transpose_propagate", transpose_propagate), ("reshape_propagate", reshape_propagate)):
        if val not in ("none", "up", "down"):
            raise ValueError("%s must be 'none', 'up' or 'down', got %r" % (name, val))
    main_passes_str = _pattern_list(
        no_nan=no_nan, all_finite=all_finite, transpose_propagate=transpose_propagate,
        reshape_propagate=reshape_propagate, max_constant_threshold=max_constant_threshold,
        excluded_passes=list(excluded_passes))
    transform_passes = ",".join([
        "enzyme-hlo-generate-td{patterns=" + main_passes_str + "}",
        "transform-interpreter",
        "enzyme-hlo-remove-transform",
    ])
    func_passes = ",".join(["canonicalize", "cse", "canonicalize", transform_passes])
    if inline:
        func_passes = "inline{default-pipeline=canonicalize max-iterations=4}" + "," + func_passes
    return func_passes


def full_optimization_pass_pipeline(**kwargs):
    """primitives.py:195-223."""
    opt_passes = optimization_passes(**kwargs)
    enzyme_pass = ('enzyme{postpasses="arith-raise{stablehlo=true},enzyme-batch-to-stablehlo,canonicalize,cse,'
                   'canonicalize,remove-unnecessary-enzyme-ops,enzyme-simplify-math,canonicalize,cse,canonicalize"}')
    propagate_down_passes = ""
    if kwargs.get("transpose_propagate", "up") == "up" or kwargs.get("reshape_propagate", "up") == "up":
        kw = dict(kwargs)
        kw.update(transpose_propagate="down", reshape_propagate="down")
        propagate_down_passes = optimization_passes(**kw)
    return ",".join([
        "mark-func-memory-effects", opt_passes, "enzyme-batch", opt_passes, enzyme_pass, opt_passes, "canonicalize",
        "remove-unnecessary-enzyme-ops", "enzyme-simplify-math", opt_passes, propagate_down_passes,
    ])


DefaultCPPPipeline = XLAPipeline()
DefaultJaXPipeline = JaXPipeline(full_optimization_pass_pipeline())


def parse_pass_pipeline(text):
    """Split an MLIR textual pass pipeline into [(pass name, option string)].
    Tolerates nested braces and quoted option values (the grammar seen in
    primitives.py:195-223 and TransformOps/GenerateApplyPatterns.cpp:98-148)."""
    out, depth, cur, quote = [], 0, [], False
    for ch in text:
        if ch == '"':
            quote = not quote
        if not quote:
            if ch == "{":
                depth += 1
            elif ch == "}":
                depth -= 1
                if depth < 0:
                    raise ValueError("unbalanced '}' in pass pipeline")
        if ch == "," and depth == 0 and not quote:
            out.append("".join(cur))
            cur = []
        else:
            cur.append(ch)
    if depth != 0 or quote:
        raise ValueError("unbalanced braces or quotes in pass pipeline")
    out.append("".join(cur))
    res = []
    for item in out:
        item = item.strip()
        if not item:
            continue
        name, _, rest = item.partition("{")
        res.append((name.strip(), rest[:-1] if rest.endswith("}") else rest))
    return res


# ---------------------------------------------------------------------------
# pytrees (dict / list / tuple of tensors), the part of jax.tree_util used at
# primitives.py:1538-1546
# ---------------------------------------------------------------------------

def tree_flatten(tree):
    leaves = []

    def walk(t):
        if isinstance(t, dict):
            return ("dict", [(k, walk(t[k])) for k in sorted(t)])
        if isinstance(t, (list, tuple)):
            return (type(t).__name__, [walk(x) for x in t])
        leaves.append(t)
        return ("leaf", None)

    return leaves, walk(tree)


def tree_unflatten(treedef, leaves):
    it = iter(leaves)

    def build(d):
        kind, sub = d
        if kind == "dict":
            return {k: build(s) for k, s in sub}
        if kind == "list":
            return [build(s) for s in sub]
        if kind == "tuple":
            return tuple(build(s) for s in sub)
        return next(it)

    return build(treedef)


def arg_activity_from_pipeline(pass_pipeline):
    """(text up to and including 'argTys=', the activities, the text after them); the list ends
    at the next space (primitives.py:502-508)."""
    start = pass_pipeline.index("argTys=")
    end = pass_pipeline.index(" ", start)
    acts = pass_pipeline[start + len("argTys="):end].split(",")
    return pass_pipeline[:start + len("argTys=")], acts, pass_pipeline[end:]


def ret_activity_from_pipeline(pass_pipeline):
    """Same for 'retTys=' (primitives.py:511-517)."""
    start = pass_pipeline.index("retTys=")
    end = pass_pipeline.index(" ", start)
    acts = pass_pipeline[start + len("retTys="):end].split(",")
    return pass_pipeline[:start + len("retTys=")], acts, pass_pipeline[end:]


def forward_mode_pipeline(pipeline_options, arg_active, n_results):
    """The pipeline `enzyme_jvp` builds for forward mode (primitives.py:1176-1203): an
    `enzyme-wrap{... mode=ForwardMode}` pass with one activity per argument (`enzyme_dup`
    where a tangent is given, `enzyme_const` for a zero tangent) and `enzyme_dup` per result,
    spliced into a pipeline that already differentiates (one more AD level) or put in front of
    one that does not."""
    arg_act = ",".join("enzyme_dup" if a else "enzyme_const" for a in arg_active)
    ret_act = ",".join(["enzyme_dup"] * n_results)
    afterad = "arith-raise{stablehlo=true},enzyme-batch-to-stablehlo, " + optimization_passes() + ", cse, canonicalize"
    newpasses = ("inline{default-pipeline=canonicalize max-iterations=4}," + optimization_passes() +
                 ", cse,enzyme-wrap{infn=main outfn= retTys=" + ret_act + " argTys=" + arg_act + " mode=ForwardMode}," + afterad)
    old = pipeline_options.pass_pipeline()
    if old != "":
        if "enzyme-wrap" in old:
            start = old.rindex("enzyme-wrap{")
            end = old.index("}", start)
            newpasses = old[:end] + afterad + newpasses + old[end:]
        else:
            newpasses = newpasses + "," + old
    return JaXPipeline(newpasses)


def reverse_mode_pipeline(forward_pipeline, ret_active):
    """The pipeline `enzyme_vjp` derives from the forward-mode one (primitives.py:1385-1419):
    the last `enzyme-wrap` pass switches to `ReverseModeCombined`, `enzyme_dup` arguments become
    `enzyme_active`, each result is `enzyme_active` where a cotangent arrives and
    `enzyme_const` where it is zero, and the cleanup passes follow."""
    passes = forward_pipeline.pass_pipeline()
    start = passes.rindex("enzyme-wrap{")
    end = passes.index("}", start)
    prev_passes, post_passes = passes[:start], passes[end + 1:]
    ad_pass = passes[start:end + 1].replace("enzyme_dup", "enzyme_active").replace("ForwardMode", "ReverseModeCombined")
    preret, _, postret = ret_activity_from_pipeline(ad_pass)
    ad_pass = preret + ",".join("enzyme_active" if a else "enzyme_const" for a in ret_active) + postret
    return JaXPipeline(prev_passes + ad_pass +
                       ",arith-raise{stablehlo=true},enzyme-batch-to-stablehlo,canonicalize, remove-unnecessary-enzyme-ops, "
                       "enzyme-simplify-math, " + optimization_passes() + ", canonicalize, cse" + post_passes)


class _EnzymeFunction:
    """What `enzyme_jax_ir(...)(func)` returns: callable for the primal; carries
    the options the reference passes to `ffi_call` (primitives.py:1571-1585)."""

    def __init__(self, func, argv, pipeline_options, jit_options, inner_jit):
        self.func = func
        self.argv = tuple(argv)
        self.pipeline_options = pipeline_options
        self.jit_options = dict(jit_options)
        self.inner_jit = inner_jit
        self.lang = LANG_MHLO
        self.__name__ = getattr(func, "__name__", "enzyme_fn")
        if pipeline_options is not None:
            if not hasattr(pipeline_options, "pass_pipeline"):
                raise TypeError("pipeline_options must be a JaXPipeline/XLAPipeline, got %r" % (pipeline_options,))
            if not pipeline_options.stablehlo_inject() and not isinstance(pipeline_options, XLAPipeline):
                raise TypeError("unsupported pipeline configuration")
            parse_pass_pipeline(pipeline_options.pass_pipeline())      # malformed strings fail here, at decoration

    def __call__(self, *args, **kwargs):
        if self.jit_options.get("print_mlir"):
            print("// enzyme_jax_ir %s lowered to targets: %s" % (self.__name__, ", ".join(sorted(ops.FFI_TARGETS))))
        return self.func(*args, **kwargs)


def enzyme_jax_ir(argv=(), pipeline_options=DefaultJaXPipeline, jit_options={}, inner_jit=True):
    """Decorator with the reference's signature (primitives.py:1528-1530)."""

    def decorator(func: Callable[..., Any]) -> Callable[..., Any]:
        return _EnzymeFunction(func, argv, pipeline_options, jit_options, inner_jit)

    return decorator


def _ad_pipeline(fn, arg_active, n_results):
    """Forward-mode pipeline for an `enzyme_jax_ir` function whose pipeline differentiates in
    MLIR, recorded as `fn.last_pipeline` (what the reference would hand to its optimizer; the
    HIP path reads only the activities from it)."""
    if not isinstance(fn, _EnzymeFunction) or fn.pipeline_options is None or not fn.pipeline_options.mlir_ad():
        return None
    fwd = forward_mode_pipeline(fn.pipeline_options, arg_active, n_results)
    fn.last_pipeline = fwd
    return fwd


def vjp(fn, *args):
    """(primals_out, f_vjp) like `jax.vjp`: `f_vjp(cotangents)` returns one
    cotangent pytree per positional argument (None for integer leaves and for
    leaves the result does not depend on... those get zeros, like the reference's
    `make_mlir_zero`, primitives.py:487-499,741)."""
    leaves, treedef = tree_flatten(args)
    with ops.Tape() as tape:
        out = fn(*args)
    out_leaves, out_def = tree_flatten(out)
    active = [isinstance(l, torch.Tensor) and l.is_floating_point() for l in leaves]
    forward = _ad_pipeline(fn, active, len(out_leaves))

    def f_vjp(cotangents):
        ct_leaves, ct_def = tree_flatten(cotangents)
        if len(ct_leaves) != len(out_leaves):
            raise ValueError("cotangent tree has %d leaves, result has %d" % (len(ct_leaves), len(out_leaves)))
        if forward is not None:
            fn.last_pipeline = reverse_mode_pipeline(forward, [c is not None for c in ct_leaves])
        wrt = [l for l in leaves if isinstance(l, torch.Tensor) and l.is_floating_point()]
        grads = tape.backward(out_leaves, ct_leaves, wrt)
        it = iter(grads)
        full = []
        for l in leaves:
            if isinstance(l, torch.Tensor) and l.is_floating_point():
                g = next(it)
                full.append(torch.zeros_like(l) if g is None else g)
            else:
                full.append(None)
        return tree_unflatten(treedef, full)

    return out, f_vjp


def jvp(fn, primals, tangents):
    """(primals_out, tangents_out) like `jax.jvp` (reference: enzyme_jvp,
    primitives.py:1147-1245): `tangents` mirrors `primals`; a None leaf (and every
    integer leaf) is a zero tangent.  Results the tangents do not reach get zeros."""
    p_leaves, p_def = tree_flatten(tuple(primals))
    t_leaves, t_def = tree_flatten(tuple(tangents))
    if len(p_leaves) != len(t_leaves):
        raise ValueError("tangent tree has %d leaves, primal tree has %d" % (len(t_leaves), len(p_leaves)))
    with ops.Forward() as fwd:
        for p, t in zip(p_leaves, t_leaves):
            if t is not None:
                if not (isinstance(p, torch.Tensor) and p.is_floating_point()):
                    raise TypeError("a tangent was given for a leaf that is not a floating-point tensor")
                fwd.seed(p, t)
        out = fn(*primals)
        out_leaves, out_def = tree_flatten(out)
        _ad_pipeline(fn, [t is not None for t in t_leaves], len(out_leaves))
        t_out = []
        for o in out_leaves:
            t = fwd.get(o) if isinstance(o, torch.Tensor) else None
            t_out.append(t if t is not None else (torch.zeros_like(o) if isinstance(o, torch.Tensor) else None))
    return out, tree_unflatten(out_def, t_out)


def ffi_call(*args, out_shapes: Sequence[Any], source, fn: str = "f", argv=(), lang: int = LANG_CPP,
             pipeline_options=DefaultCPPPipeline):
    """primitives.py:1020-1038.  C++/LLVM sources need the reference's in-process
    clang + Enzyme JIT (clang_compile.cc), which is CPU-only and not part of this build."""
    raise NotImplementedError("ffi_call with C++/LLVM/MHLO source text is not supported by the HIP path; "
                              "decorate a function written with enzyme_ad.jax.ops with enzyme_jax_ir instead")


def cpp_call(*args, out_shapes: Sequence[Any], source: str, fn: str = "f", argv=(),
             pipeline_options=DefaultCPPPipeline):
    """primitives.py:1111-1127."""
    return ffi_call(*args, source=source, fn=fn, argv=argv, out_shapes=out_shapes, lang=LANG_CPP,
                    pipeline_options=pipeline_options)


def hlo_call(*args, source: str, argv=(), passes: str = ""):
    """primitives.py:1052-1108: runs function `main` of a StableHLO module given as text on the
    arguments (device tensors whose shapes and dtypes must equal the function's, as the
    reference asserts) and returns the list of its results.  The text is parsed once per
    distinct source, its llama clusters are matched to the fused kernels, and the operators
    run on the HIP kernels with their differentiation rules, so `jvp` / `vjp` of a function
    that calls `hlo_call` work.  `passes` is parsed for validity only: the HIP path has no
    MLIR optimizer."""
    from . import stablehlo

    if passes:
        parse_pass_pipeline(passes)
    leaves, _ = tree_flatten(args)
    exe = stablehlo.compile_text(source)
    in_tys, _ = exe.signature("main")
    if len(leaves) != len(in_tys):
        raise AssertionError("main takes %d arguments, %d given" % (len(in_tys), len(leaves)))
    return exe.run(leaves, "main")


def optimize_module(mod, pipeline=None):
    """primitives.py:280-284 runs the MLIR optimizer over a module in place.  Here `mod` is the
    module's StableHLO text and the result is returned: constants folded, the llama clusters
    replaced by `stablehlo.custom_call @emi_*` (api_version 4, scalars in `backend_config`), the
    other operators printed back unchanged.  When the pipeline's last `enzyme-wrap` pass asks
    for `mode=ReverseModeCombined` (the string `enzyme_vjp` builds, :1385-1419) the result is
    the reverse-mode program instead: main(args..., cotangents of the active results) ->
    cotangents of the active arguments, with the clusters' adjoints as custom calls; for
    `mode=ForwardMode` (`enzyme_jvp`, :1176-1203) it is main(arg, tangent of arg, ...) ->
    (result, tangent of result, ...) with the clusters' tangent targets.  An XLA
    client with this library's FFI handlers registered can compile either; `hlo_call` runs
    them as well.  The other passes of the pipeline are parsed for validity only."""
    from . import stablehlo, stablehlo_ad

    passes = parse_pass_pipeline(full_optimization_pass_pipeline() if pipeline is None else pipeline)
    if not isinstance(mod, str):
        raise TypeError("optimize_module takes the module as StableHLO text (str); there are no MLIR module objects here")
    wraps = [opts for name, opts in passes if name == "enzyme-wrap"]
    if not wraps:
        return stablehlo.lower_to_custom_calls(mod)[0]
    wrap = "enzyme-wrap{" + wraps[-1] + " }"
    mode = re.search(r"mode=(\w+)", wrap)
    fn = re.search(r"infn=(\w+)", wrap)
    active = lambda acts: [a != "enzyme_const" for a in acts]
    if mode is not None and mode.group(1) == "ForwardMode":
        return stablehlo_ad.forward_module_text(mod, fn.group(1) if fn else "main",
                                                arg_active=active(arg_activity_from_pipeline(wrap)[1]))
    if mode is None or mode.group(1) != "ReverseModeCombined":
        raise NotImplementedError("optimize_module differentiates in mode=ForwardMode or mode=ReverseModeCombined; got %s" %
                                  (mode.group(1) if mode else "no mode"))
    return stablehlo_ad.reverse_module_text(mod, fn.group(1) if fn else "main",
                                            arg_active=active(arg_activity_from_pipeline(wrap)[1]),
                                            ret_active=active(ret_activity_from_pipeline(wrap)[1]))


def export(outfile, func, *args, argv=(), jit_options={}):
    """primitives.py:1489-1525 (export to LLVM IR); not built."""
    raise NotImplementedError("export needs the XLA-CPU/LLVM pipeline, which the HIP path does not have")
