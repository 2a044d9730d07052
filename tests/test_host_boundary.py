"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports
every symbol the headers declare; XLA-FFI handlers answer the metadata probe,
ignore non-execute stages and reject malformed call frames without launching;
the Python surface mirrors the reference's enzyme_ad.jax names."""
import ctypes as C
import os
import re

import pytest
import torch

import ffi_frames as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from enzyme_ad.jax import _native
    return _native.lib()


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(emi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib()
    names = _declared("emi.h") + _declared("emi_ffi.h")
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "libemi_hip.so does not export " + n
    assert lib.emi_abi_version() == 1
    from enzyme_ad.jax import _native
    assert set(_native.SIGNATURES) == set(_declared("emi.h"))      # the ctypes table covers emi.h exactly


def test_plain_launchers_reject_bad_arguments_before_touching_the_gpu():
    lib = _lib()
    assert lib.emi_rmsnorm_fwd(None, 16, 16, 16, 4, 8, 1e-5, 10) == 3          # f16 is not supported
    assert b"dtype" in lib.emi_last_error()
    assert lib.emi_rmsnorm_fwd(None, None, 16, 16, 4, 8, 1e-5, 11) == 3
    assert b"null" in lib.emi_last_error()
    assert lib.emi_rope(None, 16, 16, 16, 1, 4, 2, 7, 0, 11) == 3             # odd head_dim
    assert lib.emi_gemm(None, 16, 16, None, 16, 4, 4, -1, 4, 4, 4, 4, 0, 1, 16) == 3
    assert lib.emi_attn_fwd(None, 16, 16, 16, 16, 16, 1, 1, 8, 512, 4096, 4096, 512, 1.0, 1, 16) == 3
    assert b"head_dim" in lib.emi_last_error()
    assert lib.emi_swiglu_fwd(None, 8, 16, 16, 64, 11) == 3                    # misaligned pointer
    assert lib.emi_rmsnorm_bwd_workspace_bytes(32768, 4096) == (512 + 1) * 4096 * 4    # partial rows + second level
    # generic tensor operators
    i64 = lambda *xs: (C.c_int64 * len(xs))(*xs)
    assert lib.emi_map_binary(None, 99, 16, 16, 16, 8, 0, 0, 11) == 3 and b"operator" in lib.emi_last_error()
    assert lib.emi_map_unary(None, 0, 16, 16, 8, 11) == 3                      # a binary code on the unary entry point
    assert lib.emi_map_binary(None, 0, 16, 16, 16, 8, 0, 0, 5) == 3 and b"dtype" in lib.emi_last_error()
    assert lib.emi_convert(None, 16, 16, 8, 11, 12) == 3                       # f64 is not supported
    assert lib.emi_strided_copy(None, 16, 16, 9, i64(*[1] * 9), i64(*[1] * 9), 0, i64(*[1] * 9), 0, 4) == 3
    assert b"rank" in lib.emi_last_error()
    assert lib.emi_strided_copy(None, 16, 16, 1, i64(4), i64(1), 0, i64(1), 0, 3) == 3         # element size
    assert lib.emi_strided_copy(None, 16, 16, 1, i64(4), i64(-1), 0, i64(1), 0, 4) == 3        # negative stride
    assert lib.emi_strided_copy(None, None, None, 2, i64(0, 4), i64(4, 1), 0, i64(4, 1), 0, 4) == 0   # empty box: nothing to do
    assert lib.emi_compare(None, 6, 16, 16, 16, 8, 0, 0, 11) == 3 and b"direction" in lib.emi_last_error()
    assert lib.emi_compare(None, 0, 16, 16, None, 8, 0, 0, 11) == 3 and b"null" in lib.emi_last_error()
    assert lib.emi_select(None, 16, 16, 16, 16, 8, 0, 0, 0, 12) == 3 and b"dtype" in lib.emi_last_error()
    assert lib.emi_reduce(None, 2, 16, 16, None, 0, 4, 4, 1, 11) == 3 and b"add or max" in lib.emi_last_error()
    assert lib.emi_reduce(None, 0, 16, 16, None, 0, 70000, 4, 2, 11) == 3      # too many outer slices for the column form
    assert lib.emi_reduce(None, 0, 16, 16, None, 0, 4, 0, 1, 11) == 3          # empty reduction
    assert lib.emi_reduce_workspace_bytes(32768, 4096, 1, 16) == 0             # plenty of rows: one stage
    assert lib.emi_reduce_workspace_bytes(1, 1 << 27, 1, 16) == 2048 * 4       # full sum: 2048 fp32 partials
    assert lib.emi_reduce_workspace_bytes(1, 32768, 4096, 11) == 64 * 4096 * 4    # column sum: 4 strips x 64 bands of 512 rows, a block per CU
    # split-K partials of the GEMM: none where the 256-tile kernel fills the chip, four planes for the classifier adjoint of
    # a small model in the NT bf16 form (96 tiles of 256, K = 32000), none for the same shape in another layout or in fp32
    assert lib.emi_gemm_workspace_bytes(16384, 4096, 4096, 0, 1, 16) == 0
    assert lib.emi_gemm_workspace_bytes(8192, 768, 32000, 0, 1, 16) == 4 * 8192 * 768 * 4
    assert lib.emi_gemm_workspace_bytes(8192, 768, 32000, 0, 0, 16) == 0
    assert lib.emi_gemm_workspace_bytes(8192, 768, 32000, 0, 1, 11) == 0


def _handler(name):
    lib = _lib()
    fn = getattr(lib, name)
    fn.restype, fn.argtypes = C.c_void_p, [C.POINTER(F.CallFrame)]
    return fn


def test_ffi_metadata_probe_and_stages():
    xla = F.FakeXla()
    md = F.Metadata(C.sizeof(F.Metadata), F.ApiVersion(0, None, -1, -1), 0)
    ext = F.MetadataExt(F.ExtBase(C.sizeof(F.MetadataExt), 1, None), C.pointer(md))
    cf = xla.frame([], [])
    cf.extension_start = C.cast(C.pointer(ext), C.POINTER(F.ExtBase))
    assert _handler("emi_gemm_ffi")(C.byref(cf)) is None
    assert (md.api_version.major, md.api_version.minor) == (0, 1) and md.api_version.struct_size == C.sizeof(F.ApiVersion)
    for stage in (0, 1, 2):                                  # instantiate / prepare / initialize do nothing
        assert _handler("emi_attn_fwd_ffi")(C.byref(xla.frame([], [], stage=stage))) is None
    assert xla.errors == []


@pytest.mark.parametrize("name,args,rets,attrs,needle", [
    ("emi_rmsnorm_fwd_ffi", [(F.F32, [4, 8]), (F.F32, [7])], [(F.F32, [4, 8])], {"eps": (F.F32, 1e-5)}, "gamma"),
    ("emi_rmsnorm_fwd_ffi", [(F.F32, [4, 8]), (F.BF16, [8])], [(F.F32, [4, 8])], {"eps": (F.F32, 1e-5)}, "dtype"),
    ("emi_rmsnorm_fwd_ffi", [(F.F32, [4, 8]), (F.F32, [8])], [(F.F32, [4, 8])], {}, "eps"),
    ("emi_rmsnorm_fwd_ffi", [(F.F32, [4, 8])], [(F.F32, [4, 8])], {"eps": (F.F32, 1e-5)}, "operand"),
    ("emi_rmsnorm_bwd_ffi", [(F.F32, [4, 8]), (F.F32, [8]), (F.F32, [4, 8])], [(F.F32, [4, 8]), (F.F32, [8]), (F.U8, [16])],
     {"eps": (F.F32, 1e-5)}, "workspace"),
    ("emi_rope_ffi", [(F.BF16, [2, 16, 4, 64]), (F.F32, [16, 16, 2])], [(F.BF16, [2, 16, 4, 64])], {}, "table"),
    ("emi_gemm_ffi", [(F.BF16, [8, 16]), (F.BF16, [24, 8])], [(F.BF16, [8, 8])], {"trans_b": (F.PRED, 1)}, "contraction"),
    ("emi_gemm_ffi", [(F.BF16, [8, 16]), (F.BF16, [8, 16])], [(F.BF16, [8, 9])], {"trans_b": (F.PRED, 1)}, "C (and R)"),
    ("emi_attn_fwd_ffi", [(F.BF16, [1, 2, 64, 128])] * 3, [(F.BF16, [1, 2, 64, 128]), (F.F32, [1, 2, 63])],
     {"scale": (F.F32, 0.1), "causal": (F.PRED, 1)}, "lse"),
    ("emi_attn_fwd_ffi", [(F.BF16, [1, 2, 64, 128])] * 3, [(F.BF16, [1, 2, 64, 128]), (F.F32, [1, 2, 64])],
     {"causal": (F.PRED, 1)}, "scale"),
    ("emi_attn_bwd_ffi", [(F.BF16, [1, 2, 64, 128])] * 4 + [(F.F32, [1, 2, 64]), (F.BF16, [1, 2, 64, 128])],
     [(F.BF16, [1, 2, 64, 128])] * 3 + [(F.U8, [8])], {"scale": (F.F32, 0.1)}, "workspace"),
    ("emi_attn_step_fwd_ffi", [(F.F32, [1, 6, 48]), (F.F32, [1, 9, 6, 48]), (F.F32, [1, 9, 6, 48])],
     [(F.F32, [1, 6, 48]), (F.F32, [1, 6]), (F.U8, [8])], {"scale": (F.F32, 0.1)}, "workspace"),
    ("emi_attn_step_fwd_ffi", [(F.F32, [1, 6, 48]), (F.F32, [1, 9, 5, 48]), (F.F32, [1, 9, 5, 48])],
     [(F.F32, [1, 6, 48]), (F.F32, [1, 6]), (F.U8, [4096])], {"scale": (F.F32, 0.1)}, "head_dim"),
    ("emi_attn_step_bwd_ffi", [(F.F32, [1, 6, 48]), (F.F32, [1, 9, 6, 48]), (F.F32, [1, 9, 6, 48]), (F.F32, [1, 6, 48]),
                               (F.F32, [1, 7]), (F.F32, [1, 6, 48])],
     [(F.F32, [1, 6, 48]), (F.F32, [1, 9, 6, 48]), (F.F32, [1, 9, 6, 48]), (F.U8, [4096])], {"scale": (F.F32, 0.1)}, "lse"),
    ("emi_rmsnorm_jvp_ffi", [(F.F32, [4, 8]), (F.F32, [8]), (F.F32, [4, 8]), (F.F32, [7])], [(F.F32, [4, 8])],
     {"eps": (F.F32, 1e-5)}, "tgamma"),
    ("emi_attn_jvp_ffi", [(F.BF16, [1, 2, 64, 128])] * 3 + [(F.F32, [1, 2, 64])] + [(F.BF16, [1, 2, 64, 128])] * 3,
     [(F.BF16, [1, 2, 64, 128])], {"causal": (F.PRED, 1)}, "scale"),
    ("emi_embedding_fwd_ffi", [(F.S64, [3]), (F.F32, [10, 4])], [(F.F32, [3, 4])], {}, "s32"),
    ("emi_swiglu_bwd_ffi", [(F.F32, [8])] * 3, [(F.F32, [8]), (F.F32, [9])], {}, "shape"),
    ("emi_gemm_rope_ffi", [(F.BF16, [32, 16]), (F.BF16, [64, 16]), (F.BF16, [16, 32, 2])], [(F.BF16, [32, 64])], {}, "table"),
    ("emi_gemm_rope_ffi", [(F.BF16, [32, 16]), (F.BF16, [64, 24]), (F.F32, [16, 32, 2])], [(F.BF16, [32, 64])], {}, "contraction"),
    ("emi_gemm_rope_ffi", [(F.BF16, [32, 16]), (F.BF16, [64, 16]), (F.F32, [16, 32, 2])], [(F.BF16, [32, 60])], {}, "y must be"),
    ("emi_gemm_swiglu_fwd_ffi", [(F.BF16, [32, 16]), (F.BF16, [64, 16]), (F.BF16, [32, 48])], [(F.BF16, [32, 64])] * 2, {}, "a, b, g"),
    ("emi_gemm_swiglu_bwd_ffi", [(F.BF16, [32, 16]), (F.BF16, [64, 16]), (F.BF16, [32, 64]), (F.F32, [32, 64])],
     [(F.BF16, [32, 64])] * 2, {}, "dtype"),
    ("emi_attn_bwd_rope_ffi", [(F.BF16, [1, 64, 2, 128])] * 4 + [(F.F32, [1, 2, 64]), (F.BF16, [1, 64, 2, 128]), (F.F32, [64, 32, 2])],
     [(F.BF16, [1, 64, 2, 128])] * 3 + [(F.U8, [1024])], {"scale": (F.F32, 0.1), "bshd": (F.PRED, 1)}, "table"),
    ("emi_attn_bwd_rope_ffi", [(F.BF16, [1, 64, 2, 128])] * 4 + [(F.F32, [1, 2, 64]), (F.BF16, [1, 64, 2, 128]), (F.F32, [64, 64, 2])],
     [(F.BF16, [1, 64, 2, 128])] * 3 + [(F.U8, [8])], {"scale": (F.F32, 0.1), "bshd": (F.PRED, 1)}, "workspace"),
])
def test_ffi_rejects_malformed_frames(name, args, rets, attrs, needle):
    xla = F.FakeXla()
    cf = xla.frame([xla.buffer(*a) for a in args], [xla.buffer(*r) for r in rets], attrs)
    err = _handler(name)(C.byref(cf))
    assert err is not None and len(xla.errors) == 1
    code, msg = xla.errors[0]
    assert code == F.INVALID_ARGUMENT and needle in msg, msg


def test_ffi_null_buffer_and_missing_stream_getter():
    xla = F.FakeXla()
    cf = xla.frame([xla.buffer(F.F32, [8], data=None), xla.buffer(F.F32, [8])], [xla.buffer(F.F32, [8])])
    assert _handler("emi_add_ffi")(C.byref(cf)) is not None and "null" in xla.errors[-1][1]
    xla.api.struct_size = 48                                  # an API table that ends before Stream_Get
    cf = xla.frame([xla.buffer(F.F32, [8]), xla.buffer(F.F32, [8])], [xla.buffer(F.F32, [8])])
    assert _handler("emi_add_ffi")(C.byref(cf)) is not None and "Stream_Get" in xla.errors[-1][1]


def test_ffi_registration_lists_all_targets_for_rocm():
    lib = _lib()
    lib.emi_ffi_target_name.restype = C.c_char_p
    lib.emi_ffi_target_handler.restype = C.c_void_p
    n = lib.emi_ffi_target_count()
    names = [lib.emi_ffi_target_name(i).decode() for i in range(n)]
    assert n == 26 and "emi_gemm_rope" in names and "emi_attn_bwd_rope" in names and "emi_gemm_swiglu_bwd" in names and "emi_gemm_grouped" in names and "emi_cross_entropy_bwd" in names and "emi_attn_bwd" in names and "emi_attn_step_bwd" in names and "emi_attn_jvp" in names and all(lib.emi_ffi_target_handler(i) for i in range(n))
    from enzyme_ad.jax import ops
    used = {t for fwd, bwd in ops.FFI_TARGETS.values() for t in (fwd,) + tuple(bwd)}
    used |= {t for ts in ops.FFI_TANGENT_TARGETS.values() for t in ts}
    assert used <= set(names)                                 # every target the lowering table names has a handler
    xla = F.FakeXla()
    lib.emi_register_ffi.argtypes = [C.POINTER(F.Api)]
    assert lib.emi_register_ffi(C.byref(xla.api)) == 0
    assert sorted(r[0] for r in xla.registered) == sorted(names) and {r[1] for r in xla.registered} == {"ROCM"}
    assert lib.emi_register_ffi(C.byref(xla.api)) == 0 and len(xla.registered) == n     # once per process
    assert lib.emi_register_ffi(None) == 3


def test_python_surface_matches_reference_names():
    import enzyme_ad.jax as ej
    for name in ["cpp_call", "ffi_call", "hlo_call", "enzyme_jax_ir", "optimize_module", "export", "XLAPipeline",
                 "JaXPipeline", "full_optimization_pass_pipeline", "optimization_passes"]:   # __init__.py:1-12
        assert hasattr(ej, name), name
    p = ej.JaXPipeline("inline,enzyme-wrap{infn=main outfn= retTys=enzyme_dup argTys=enzyme_dup mode=ForwardMode},cse")
    assert p.mlir_ad() and p.stablehlo_inject() and p.ad_level() == 1 and p.pass_pipeline().startswith("inline")
    x = ej.XLAPipeline("out.ll")
    assert not x.mlir_ad() and not x.stablehlo_inject() and x.export_llvm() == "out.ll" and x.pass_pipeline() == ""
    full = ej.full_optimization_pass_pipeline(inline=False, no_nan=True)
    parsed = ej.parse_pass_pipeline(full)
    names = [n for n, _ in parsed]
    assert names[0] == "mark-func-memory-effects" and "enzyme-batch" in names and "enzyme" in names
    enz = dict(parsed)["enzyme"]
    assert enz.startswith('postpasses="arith-raise{stablehlo=true}')            # nested braces inside quotes survive
    assert "inline" not in names and "no_nan<1>" in full
    assert ej.optimization_passes().startswith("inline{default-pipeline=canonicalize max-iterations=4},canonicalize,cse")
    with pytest.raises(ValueError):
        ej.optimization_passes(transpose_propagate="sideways")
    with pytest.raises(ValueError):
        ej.parse_pass_pipeline("a{b")
    with pytest.raises(TypeError):
        ej.enzyme_jax_ir(pipeline_options="not a pipeline")(lambda x: x)
    f = ej.enzyme_jax_ir(argv=("-O3",), pipeline_options=ej.JaXPipeline(), jit_options={"print_mlir": False}, inner_jit=False)(lambda x: x)
    assert f(3) == 3 and f.argv == ("-O3",)
    with pytest.raises(NotImplementedError):
        ej.cpp_call(out_shapes=[], source="void f(){}")
    with pytest.raises(ValueError):                     # a module without a function
        ej.hlo_call(source="module {}")
    with pytest.raises(RuntimeError):                   # host tensors: there is no CPU path
        ej.hlo_call(torch.ones(2), source="func.func @main(%a: tensor<2xf32>) -> tensor<2xf32> {\n return %a : tensor<2xf32>\n}")
    with pytest.raises(TypeError):                      # a tangent for a leaf that is not a floating-point tensor
        ej.jvp(f, (1,), (1,))
    out, tangent = ej.jvp(f, (3,), (None,))             # jax.jvp shape of the result: (primals_out, tangents_out)
    assert out == 3 and tangent is None


def test_operators_refuse_host_tensors():
    import torch
    from enzyme_ad.jax import ops
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.rmsnorm(torch.zeros(2, 8), torch.ones(8))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.gemm(torch.zeros(2, 8), torch.zeros(8, 2))


def test_tape_fan_in_without_gpu():
    """The tape's bookkeeping, exercised with a stub operator (no kernels run)."""
    import torch
    from enzyme_ad.jax import ops
    a, b = torch.ones(3), torch.ones(3)
    with ops.Tape() as tape:
        y = a * 2
        ops.Tape.record((a,), y, lambda c, acc: (c * 2 if acc[0] is None else acc[0] + c * 2,))
        z = y + a
        ops.Tape.record((y, a), z, lambda c, acc: (c if acc[0] is None else acc[0] + c, c if acc[1] is None else acc[1] + c))
    ga, gb = tape.backward([z], [torch.ones(3)], [a, b])
    assert torch.equal(ga, torch.full((3,), 3.0)) and gb is None


def test_activity_pipeline_strings_round_trip():
    """The strings `enzyme_jvp` / `enzyme_vjp` build (primitives.py:502-517,1176-1203,1385-1419):
    activities per argument and result, ForwardMode -> ReverseModeCombined, and the splice into
    a pipeline that already differentiates."""
    from enzyme_ad.jax import primitives as P

    fwd = P.forward_mode_pipeline(P.JaXPipeline(), [True, False, True], 2)
    s = fwd.pass_pipeline()
    wrap = "enzyme-wrap{infn=main outfn= retTys=enzyme_dup,enzyme_dup argTys=enzyme_dup,enzyme_const,enzyme_dup mode=ForwardMode}"
    assert wrap in s and s.startswith("inline{default-pipeline=canonicalize max-iterations=4},")
    assert s.endswith(", cse, canonicalize") and fwd.ad_level() == 1
    pre, acts, post = P.arg_activity_from_pipeline(s)
    assert acts == ["enzyme_dup", "enzyme_const", "enzyme_dup"] and pre.endswith("argTys=") and post.startswith(" mode=ForwardMode}")
    assert pre + ",".join(acts) + post == s                                  # lossless split
    pre, acts, post = P.ret_activity_from_pipeline(s)
    assert acts == ["enzyme_dup", "enzyme_dup"] and pre + ",".join(acts) + post == s
    rev = P.reverse_mode_pipeline(fwd, [True, False]).pass_pipeline()
    assert ("enzyme-wrap{infn=main outfn= retTys=enzyme_active,enzyme_const argTys=enzyme_active,enzyme_const,enzyme_active "
            "mode=ReverseModeCombined}") in rev
    assert "ForwardMode" not in rev and "enzyme_dup" not in rev
    assert ",arith-raise{stablehlo=true},enzyme-batch-to-stablehlo,canonicalize, remove-unnecessary-enzyme-ops, enzyme-simplify-math, " in rev
    assert [n for n, _ in P.parse_pass_pipeline(rev)].count("enzyme-wrap") == 1
    # a user pipeline without AD is appended; one with AD gets the new pass spliced after its own
    plain = P.forward_mode_pipeline(P.JaXPipeline("canonicalize,cse"), [True], 1).pass_pipeline()
    assert plain.endswith(", cse, canonicalize,canonicalize,cse")
    twice = P.forward_mode_pipeline(fwd, [True, False, True, True, True], 4)
    assert twice.ad_level() == 2
    assert P.arg_activity_from_pipeline(twice.pass_pipeline())[1] == ["enzyme_dup", "enzyme_const", "enzyme_dup"]   # first pass kept
    with pytest.raises(ValueError):
        P.arg_activity_from_pipeline("canonicalize")


def test_vjp_and_jvp_record_the_reference_pipeline():
    import enzyme_ad.jax as ej

    f = ej.enzyme_jax_ir(pipeline_options=ej.JaXPipeline(), inner_jit=False)(lambda a, b: a)
    ej.jvp(f, (3, 4), (None, None))
    assert "argTys=enzyme_const,enzyme_const mode=ForwardMode" in f.last_pipeline.pass_pipeline()
    out, f_vjp = ej.vjp(f, 3, 4)
    assert "mode=ForwardMode" in f.last_pipeline.pass_pipeline()
    g = ej.enzyme_jax_ir(pipeline_options=ej.XLAPipeline(), inner_jit=False)(lambda a: a)     # no MLIR AD: nothing recorded
    ej.jvp(g, (3,), (None,))
    assert not hasattr(g, "last_pipeline")


def test_bench_refuses_more_than_one_gpu_and_entry_points_exist():
    """bench.py is a one-GPU program: asked for more it exits with a message instead of launching anything;
    the repository entry module exposes build() and smoke()."""
    import importlib.util
    import subprocess
    import sys as _sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([_sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
    spec = importlib.util.spec_from_file_location("graft_entry", os.path.join(root, "__graft_entry__.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert callable(mod.build) and callable(mod.smoke)
