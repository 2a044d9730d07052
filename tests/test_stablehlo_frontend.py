"""Host logic of the StableHLO text front end: the parser on the spellings MLIR prints, the
constant folder, and the cluster matcher on the llama step text (no device needed)."""
from collections import Counter

import numpy as np
import pytest

from enzyme_ad.jax.llama_text import llama_step_text

CFG = {"dim": 288, "hidden_dim": 768, "n_layers": 2, "n_heads": 6, "n_kv_heads": 6}


def test_parser_accepts_pretty_and_quoted_spellings():
    from enzyme_ad.jax import stablehlo as S

    text = '''
    // a comment
    func.func @f(%a : tensor<2x3xf32>, %b : tensor<4x2xf32>) -> tensor<3x4xf32> {
      %c = "stablehlo.dot_general"(%a, %b) {
        dot_dimension_numbers = #stablehlo.dot<
          lhs_batching_dimensions = [], rhs_batching_dimensions = [],
          lhs_contracting_dimensions = [0], rhs_contracting_dimensions = [1]>,
        precision_config = [#stablehlo<precision DEFAULT>, #stablehlo<precision DEFAULT>]
      } : (tensor<2x3xf32>, tensor<4x2xf32>) -> tensor<3x4xf32>
      %m = stablehlo.constant dense<0xFF800000> : tensor<f32>
      %r = stablehlo.reduce(%c init: %m) across dimensions = [1] : (tensor<3x4xf32>, tensor<f32>) -> tensor<3xf32>
       reducer(%x: tensor<f32>, %y: tensor<f32>)  {
        %z = stablehlo.maximum %x, %y : tensor<f32>
        stablehlo.return %z : tensor<f32>
      }
      %s = stablehlo.slice %c [0:2, 1:4:2] : (tensor<3x4xf32>) -> tensor<2x2xf32>
      %k = stablehlo.constant dense<[[1.0, 2.0], [3.0, -4.5e0]]> : tensor<2x2xf32>
      %cc = stablehlo.concatenate %s, %k, dim = 0 : (tensor<2x2xf32>, tensor<2x2xf32>) -> tensor<4x2xf32>
      %t = "stablehlo.transpose"(%cc) {permutation = array<i64: 1, 0>} : (tensor<4x2xf32>) -> tensor<2x4xf32>
      %h = stablehlo.constant dense<"0x0000803F00000040"> : tensor<2xf32>
      %bf = stablehlo.constant dense<1.500000e+00> : tensor<4xbf16>
      %q = call @g(%h) : (tensor<2xf32>) -> tensor<2xf32>
      func.return %c : tensor<3x4xf32>
    }
    func.func private @g(%a: tensor<2xf32> {mhlo.layout_mode = "default"}) -> (tensor<2xf32> {jax.result_info = ""}) {
      return %a : tensor<2xf32>
    }
    '''
    funcs = S.parse_module(text)
    ops = {o.results[0]: o for o in funcs["f"].ops if o.results}
    assert ops["%c"].attrs == {"batch_a": [], "batch_b": [], "contract_a": [0], "contract_b": [1]}
    assert ops["%m"].attrs["value"] == -np.inf
    assert ops["%r"].attrs == {"dims": [1], "body": "maximum"}
    assert ops["%s"].attrs == {"start": [0, 1], "limit": [2, 4], "stride": [1, 2]}
    assert np.array_equal(ops["%k"].attrs["value"], [[1.0, 2.0], [3.0, -4.5]])
    assert ops["%t"].attrs == {"perm": [1, 0]} and ops["%t"].types[0].shape == (2, 4)
    assert np.array_equal(ops["%h"].attrs["value"], [1.0, 2.0])
    assert ops["%bf"].types[0].dtype == "bf16" and ops["%q"].attrs["callee"] == "g"
    assert funcs["g"].args[0][1].shape == (2,)


def test_parser_errors_name_the_line_and_the_operator():
    from enzyme_ad.jax import stablehlo as S

    with pytest.raises(S.ParseError, match="line 2"):
        S.parse_module("func.func @main(%a: tensor<2xf32>) -> tensor<2xf32> {\n  %b = stablehlo.add %a %a : tensor<2xf32>\n}")
    with pytest.raises(NotImplementedError, match="stablehlo.erf_inv"):
        S.parse_module("func.func @main(%a: tensor<f32>) -> tensor<f32> {\n %b = stablehlo.erf_inv %a : tensor<f32>\n return %b : tensor<f32>\n}")
    with pytest.raises(S.ParseError):
        S.parse_module("func.func @main(%a: tensor<?xf32>) -> tensor<2xf32> {\n return %a : tensor<2xf32>\n}")
    with pytest.raises(S.ParseError):
        S.parse_module("module {}")


def test_llama_text_clusters_are_matched():
    from enzyme_ad.jax import stablehlo as S

    text, order = llama_step_text(CFG, pos=3)
    exe = S.Executable(text)
    L = CFG["n_layers"]
    assert exe.fused == {"rmsnorm": 2 * L + 1, "swiglu": L, "rope": 2 * L, "softmax_dot": 6 * L, "attention_step": L,
                         "linear": 7 * L}
    left = Counter(o.name for o in exe.funcs["main"].ops)
    # what stays generic: weight slices / reshapes and the two cache appends per layer; the seven
    # projections per layer are emi.linear, two of them with the residual add folded in
    assert left["emi.linear"] == 7 * L and left["concatenate"] == 2 * L and "add" not in left and "dot_general" not in left
    assert sum(len(o.operands) == 3 for o in exe.funcs["main"].ops if o.name == "emi.linear") == 2 * L
    assert not any(k in left for k in ("exponential", "reduce", "sqrt", "divide", "multiply", "broadcast_in_dim", "constant"))
    att = [o for o in exe.funcs["main"].ops if o.name == "emi.attention_step"][0]
    assert att.attrs["heads"] == 6 and att.attrs["rows"] == 4 and abs(att.attrs["scale"] - 1 / np.sqrt(48)) < 1e-7
    rope = [o for o in exe.funcs["main"].ops if o.name == "emi.rope"][0]
    assert rope.attrs["table"].shape == (144, 2)
    # unfused: only the constant folder ran (sqrt of the head size became a constant)
    plain = S.Executable(text, fuse=False)
    names = Counter(o.name for o in plain.funcs["main"].ops)
    assert plain.fused == {} and names["sqrt"] == 2 * L + 1 and names["exponential"] == 7 * L


def test_run_list_joins_the_sub_blocks_of_a_layer():
    """On the list the executable walks, projections + rotation + attention and projections + SwiGLU + projection of a
    batched layer are the two operators that apply the elementwise parts in the epilogues; the function's own
    operator list (what is printed and differentiated symbolically) keeps the separate clusters."""
    from enzyme_ad.jax import stablehlo as S
    from enzyme_ad.jax.llama_text import llama_layer_text, llama_model_text

    text, _ = llama_layer_text({"dim": 128, "hidden_dim": 352, "n_heads": 2}, 2, 40, "bf16")
    f = S.Executable(text).funcs["main"]
    run = Counter(o.name for o in f.run_ops)
    assert run == Counter({"emi.rmsnorm_rows": 2, "emi.attention_block": 1, "emi.linear": 1, "emi.ffn": 1, "return": 1})
    own = Counter(o.name for o in f.ops)
    assert own["emi.rope_rows"] == 2 and own["emi.swiglu"] == 1 and "emi.ffn" not in own
    blk = [o for o in f.run_ops if o.name == "emi.attention_block"][0]
    assert blk.attrs["heads"] == 2 and blk.attrs["causal"] and blk.attrs["table"].shape == (40, 32, 2) and len(blk.operands) == 4
    ffn = [o for o in f.run_ops if o.name == "emi.ffn"][0]
    assert len(ffn.operands) == 5                                      # x, w1, w3, w2 and the residual
    # whole model: every layer's blocks, the weights as in-place selects of the stacked arguments
    cfg = {"dim": 64, "hidden_dim": 176, "n_layers": 3, "n_heads": 2, "vocab_size": 100}
    text, _ = llama_model_text(cfg, 2, 24, "bf16", loss="gather")
    run = Counter(o.name for o in S.Executable(text).funcs["main"].run_ops)
    assert run["emi.ffn"] == 3 and run["emi.attention_block"] == 3 and run["emi.select"] == 27 and "emi.swiglu" not in run


def test_optimize_module_prints_the_fused_epilogue_targets():
    """The batched layer as optimize_module prints it: q and k projections stored rotated (`emi_gemm_rope`), the SwiGLU
    in the epilogue of the w3 product (`emi_gemm_swiglu_fwd`); the reverse program turns dq / dk back inside the
    attention adjoint (`emi_attn_bwd_rope`, no `emi_rope`) and runs the SwiGLU adjoint in the epilogue of dy . w2
    (`emi_gemm_swiglu_bwd` on the transposed down projection, no `emi_swiglu_bwd`).  The forward-mode program keeps the
    separate clusters (their tangent targets)."""
    import re
    from enzyme_ad.jax import optimize_module, primitives as P, stablehlo as S
    from enzyme_ad.jax.llama_text import llama_layer_text

    text, _ = llama_layer_text({"dim": 128, "hidden_dim": 352, "n_heads": 2}, 2, 40, "bf16")
    calls = lambda t: re.findall(r"custom_call @(\w+)", t)
    low = optimize_module(text)
    assert calls(low) == ["emi_rmsnorm_fwd", "emi_gemm_rope", "emi_gemm_rope", "emi_gemm", "emi_attn_fwd", "emi_gemm", "emi_rmsnorm_fwd",
                          "emi_gemm", "emi_gemm_swiglu_fwd", "emi_gemm"]
    fwd_pipe = P.forward_mode_pipeline(P.JaXPipeline(), [True] * 10, 1)
    rev = optimize_module(text, P.reverse_mode_pipeline(fwd_pipe, [True]).pass_pipeline())
    rc = Counter(calls(rev))
    assert rc["emi_attn_bwd_rope"] == 1 and rc["emi_gemm_swiglu_bwd"] == 1 and rc["emi_rmsnorm_bwd"] == 2
    assert "emi_rope" not in rc and "emi_swiglu_bwd" not in rc and "emi_attn_bwd" not in rc
    assert "stablehlo.transpose" in rev                                   # the down projection, transposed for the fused adjoint
    # the adjoint products of sibling projections, as the tape issues them: dxb = dq . wq + dk . wk + dv . wv as one summed
    # launch and dwq, dwk, dwv as one grouped launch; the same for the pair w1 / w3
    grouped = sorted(re.findall(r"@emi_gemm_grouped\(.*?count = (\d+).*?sum = (\w+).*?trans_a = (\w+)", rev))
    assert grouped == [("2", "false", "true"), ("2", "true", "false"), ("3", "false", "true"), ("3", "true", "false")], grouped
    line = [l for l in rev.splitlines() if "@emi_attn_bwd_rope" in l][0]
    assert line.count("tensor<2x40x2x64xbf16>") >= 8 and "tensor<40x32x2xf32>" in line and "bshd = true" in line
    fw = Counter(calls(optimize_module(text, fwd_pipe.pass_pipeline())))
    assert fw["emi_rope"] == 4 and fw["emi_swiglu_jvp"] == 1 and fw["emi_attn_jvp"] == 1 and "emi_gemm_rope" not in fw
    for t in (low, rev):
        S.Executable(t, fuse=False)                                       # the printed text parses back


def test_matcher_leaves_clusters_with_outside_uses_alone():
    from enzyme_ad.jax import stablehlo as S

    # the sigmoid is also returned: the swiglu cluster must stay unfused
    text = """
    func.func @main(%a: tensor<8xf32>, %b: tensor<8xf32>) -> (tensor<8xf32>, tensor<8xf32>) {
      %s = stablehlo.logistic %a : tensor<8xf32>
      %m = stablehlo.multiply %a, %s : tensor<8xf32>
      %r = stablehlo.multiply %m, %b : tensor<8xf32>
      return %r, %s : tensor<8xf32>, tensor<8xf32>
    }"""
    assert S.Executable(text).fused.get("swiglu", 0) == 0
    fused = S.Executable(text.replace("return %r, %s : tensor<8xf32>, tensor<8xf32>", "return %r, %r : tensor<8xf32>, tensor<8xf32>"))
    assert fused.fused["swiglu"] == 1
    # a "rotation" constant that is not a rotation is not a rope cluster
    bad = """
    func.func @main(%x: tensor<4xf32>) -> tensor<4xf32> {
      %R = stablehlo.constant dense<[[[1.0, 2.0], [3.0, 4.0]], [[1.0, 0.0], [0.0, 1.0]]]> : tensor<2x2x2xf32>
      %v = stablehlo.reshape %x : (tensor<4xf32>) -> tensor<2x2xf32>
      %d = stablehlo.dot_general %R, %v, batching_dims = [0] x [0], contracting_dims = [2] x [1] : (tensor<2x2x2xf32>, tensor<2x2xf32>) -> tensor<2x2xf32>
      %y = stablehlo.reshape %d : (tensor<2x2xf32>) -> tensor<4xf32>
      return %y : tensor<4xf32>
    }"""
    assert S.Executable(bad).fused.get("rope", 0) == 0


def test_optimize_module_prints_typed_ffi_custom_calls():
    """optimize_module: clusters come back as stablehlo.custom_call @emi_* in the typed-FFI wire
    format (api_version 4, scalars in backend_config, row-major layouts); the printed module
    parses again and printing it once more changes nothing."""
    import enzyme_ad.jax as ej
    from enzyme_ad.jax import stablehlo as S

    text, order = llama_step_text(dict(CFG, n_layers=1), pos=3)
    low = ej.optimize_module(text)
    calls = [l.strip() for l in low.splitlines() if "stablehlo.custom_call" in l]
    assert Counter(l.split("@")[1].split("(")[0] for l in calls) == {"emi_rmsnorm_fwd": 3, "emi_rope": 2, "emi_attn_step_fwd": 1, "emi_swiglu_fwd": 1,
                                                                     "emi_gemm": 7}
    assert all("api_version = 4 : i32" in l and "backend_config = {" in l and "operand_layouts = [" in l for l in calls)
    rms = [l for l in calls if "emi_rmsnorm_fwd" in l][0]
    assert "backend_config = {eps = 9.999999747e-06 : f32}" in rms
    assert "operand_layouts = [dense<[1, 0]> : tensor<2xindex>, dense<0> : tensor<1xindex>]" in rms
    assert ": (tensor<1x288xf32>, tensor<288xf32>) -> tensor<1x288xf32>" in rms
    att = [l for l in calls if "emi_attn_step_fwd" in l][0]
    assert ":3 = stablehlo.custom_call" in att and "scale = 1.443375647e-01 : f32" in att or "scale = 1.4433756" in att
    assert "-> (tensor<1x6x48xf32>, tensor<1x6xf32>, tensor<1200xi8>)" in att          # o, lse, workspace (1 split of 512 keys)
    for gone in ("stablehlo.exponential", "stablehlo.sqrt", "stablehlo.reduce", "stablehlo.divide"):
        assert gone not in low
    again = S.parse_module(low)
    ccs = [o for o in again["main"].ops if o.name == "custom_call"]
    assert ccs[0].attrs["target"] == "emi_rmsnorm_fwd" and abs(ccs[0].attrs["config"]["eps"] - 1e-5) < 1e-11
    assert [o.attrs["config"] for o in ccs if o.attrs["target"] == "emi_rope"][0] == {"inverse": False}
    assert S.print_module(again) == low
    with pytest.raises(TypeError):
        ej.optimize_module(object())
    with pytest.raises(ValueError):
        ej.optimize_module(text, pipeline="a{b")


def _ops_of(text, fn="main"):
    from enzyme_ad.jax import stablehlo as S
    return [(o.name, tuple(o.operands), {k: v for k, v in o.attrs.items() if k != "value"}) for o in S.parse_module(text)[fn].ops]


def test_symbolic_reverse_mode_has_the_reference_ir_form():
    """The reverse programs the reference's lit tests expect (their REVERSE check lines, minus
    the additions of zero constants and identity transposes): dot_general.mlir:25-37 and
    divide.mlir:21-27."""
    from enzyme_ad.jax import stablehlo_ad as A

    dot = """func.func @main(%a: tensor<2x3xf32>, %b: tensor<4x2xf32>) -> tensor<3x4xf32> {
      %c = stablehlo.dot_general %a, %b, contracting_dims = [0] x [1] : (tensor<2x3xf32>, tensor<4x2xf32>) -> tensor<3x4xf32>
      return %c : tensor<3x4xf32>
    }"""
    ops = _ops_of(A.reverse_module_text(dot))
    assert [o[0] for o in ops] == ["dot_general", "transpose", "dot_general", "return"]
    assert ops[0][1] == ("%ct0", "%b") and ops[0][2] == {"batch_a": [], "batch_b": [], "contract_a": [1], "contract_b": [0]}
    assert ops[1][2] == {"perm": [1, 0]}
    assert ops[2][1] == ("%ct0", "%a") and ops[2][2] == {"batch_a": [], "batch_b": [], "contract_a": [0], "contract_b": [1]}
    div = """func.func @main(%a: tensor<2xf32>, %b: tensor<2xf32>) -> tensor<2xf32> {
      %c = stablehlo.divide %a, %b : tensor<2xf32>
      return %c : tensor<2xf32>
    }"""
    ops = _ops_of(A.reverse_module_text(div))
    # %0 = ct / b; %1 = a / b; %2 = %0 * %1; %3 = -%2; return %0, %3
    assert sorted(o[0] for o in ops) == ["divide", "divide", "multiply", "negate", "return"]
    by = {o[0]: o for o in ops if o[0] in ("multiply", "negate", "return")}
    q = [o for o in ops if o[0] == "divide" and o[1][0] == "%ct0"]
    assert len(q) == 1 and q[0][1][1] == "%b" and by["multiply"][1][1] == "%c"
    # activities: an inactive argument gets no result, an inactive result no cotangent argument
    rev = A.reverse_module_text(div, arg_active=[False, True])
    f = __import__("enzyme_ad.jax.stablehlo", fromlist=["x"]).parse_module(rev)["main"]
    assert len(f.result_types) == 1 and [a for a, _ in f.args] == ["%a", "%b", "%ct0"]
    # maximum: a compare and two selects (ties to the first operand, maximum.mlir:25-34)
    ops = _ops_of(A.reverse_module_text("""func.func @main(%a: tensor<2xf32>, %b: tensor<2xf32>) -> tensor<2xf32> {
      %c = stablehlo.maximum %a, %b : tensor<2xf32>
      return %c : tensor<2xf32>
    }"""))
    assert sorted(o[0] for o in ops) == ["compare", "constant", "return", "select", "select"]
    assert [o[2] for o in ops if o[0] == "compare"] == [{"direction": "GE"}]


def test_symbolic_reverse_of_the_llama_step_calls_the_adjoint_targets():
    from enzyme_ad.jax import stablehlo as S, stablehlo_ad as A

    text, order = llama_step_text(dict(CFG, n_layers=1), pos=3)
    rev = A.reverse_module_text(text)
    f = S.parse_module(rev)["main"]
    targets = Counter(o.attrs["target"] for o in f.ops if o.name == "custom_call")
    # forward values the adjoints need are recomputed (the final RMSNorm's output is not needed)
    assert targets == {"emi_rope": 4, "emi_rmsnorm_bwd": 3, "emi_rmsnorm_fwd": 2, "emi_attn_step_fwd": 1, "emi_swiglu_fwd": 1,
                       "emi_swiglu_bwd": 1, "emi_attn_step_bwd": 1, "emi_gemm": 7 + 14}      # 7 projections, dX and dW of each
    assert sorted(o.attrs["config"]["inverse"] for o in f.ops if o.name == "custom_call" and o.attrs["target"] == "emi_rope") == \
        [False, False, True, True]
    # the seven dx = dy . W products of one token declare the scratch their kernel sums row bands in (an extra i8 result
    # of emi_gemm_workspace_bytes bytes, which the handler takes when it is there); no other product needs one
    with_ws = [o for o in f.ops if o.name == "custom_call" and o.attrs["target"] == "emi_gemm" and len(o.results) == 2]
    assert len(with_ws) == 7 and all(o.types[1].dtype == "i8" and not o.attrs["config"]["trans_a"] and not o.attrs["config"]["trans_b"]
                                     for o in with_ws)
    assert len(f.args) == len(order) + 1 and f.args[-1][1].shape == (288,)
    assert [t.shape for t in f.result_types] == [t.shape for _, t in f.args[:-1]]
    assert S.print_module(S.parse_module(rev)) == rev
    bwd = [o for o in f.ops if o.name == "custom_call" and o.attrs["target"] == "emi_attn_step_bwd"][0]
    fwd = [o for o in f.ops if o.name == "custom_call" and o.attrs["target"] == "emi_attn_step_fwd"][0]
    assert bwd.operands[3:5] == fwd.results[:2]                                  # o and lse of the forward call


def test_optimize_module_differentiates_when_the_pipeline_says_so():
    """The pipeline strings enzyme_jvp / enzyme_vjp build select the program optimize_module
    returns: lowering only, or the reverse-mode program with the listed activities."""
    import enzyme_ad.jax as ej
    from enzyme_ad.jax import primitives as P, stablehlo as S

    text = """func.func @main(%a: tensor<2xf32>, %b: tensor<2xf32>) -> tensor<2xf32> {
      %c = stablehlo.divide %a, %b : tensor<2xf32>
      return %c : tensor<2xf32>
    }"""
    fwd = P.forward_mode_pipeline(P.JaXPipeline(), [False, True], 1)
    rev = P.reverse_mode_pipeline(fwd, [True])
    out = S.parse_module(ej.optimize_module(text, rev.pass_pipeline()))["main"]
    assert [a for a, _ in out.args] == ["%a", "%b", "%ct0"] and len(out.result_types) == 1      # a is enzyme_const
    assert sorted(o.name for o in out.ops) == ["divide", "divide", "multiply", "negate", "return"]
    plain = S.parse_module(ej.optimize_module(text))["main"]
    assert [o.name for o in plain.ops] == ["divide", "return"]
    # forward mode: (ta b - tb a) / b^2 with a inactive -> -(tb a) / (b b), primal last (divide.mlir:9-17)
    f = S.parse_module(ej.optimize_module(text, fwd.pass_pipeline()))["main"]
    assert [a for a, _ in f.args] == ["%a", "%b", "%t_b"] and len(f.result_types) == 2
    assert sorted(o.name for o in f.ops) == ["divide", "divide", "multiply", "multiply", "negate", "return"]
    both = S.parse_module(ej.optimize_module(text, P.forward_mode_pipeline(P.JaXPipeline(), [True, True], 1).pass_pipeline()))["main"]
    assert [a for a, _ in both.args] == ["%a", "%t_a", "%b", "%t_b"]
    assert sorted(o.name for o in both.ops) == ["divide", "divide", "multiply", "multiply", "multiply", "return", "subtract"]
    with pytest.raises(NotImplementedError, match="ForwardModeSplit"):
        ej.optimize_module(text, fwd.pass_pipeline().replace("mode=ForwardMode", "mode=ForwardModeSplit"))


def test_parser_drops_debug_locations():
    from enzyme_ad.jax import stablehlo as S

    text = """#loc = loc(unknown)
module @jit_f attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  func.func public @main(%arg0: tensor<4xf32> {mhlo.layout_mode = "default"} loc(unknown)) -> (tensor<4xf32> {jax.result_info = ""}) {
    %0 = stablehlo.multiply %arg0, %arg0 : tensor<4xf32> loc(#loc2)
    %1 = call @inner(%0) : (tensor<4xf32>) -> tensor<4xf32> loc(#loc3)
    return %1 : tensor<4xf32> loc(#loc)
  } loc(#loc)
  func.func private @inner(%arg0: tensor<4xf32> loc("x(1)"(callsite("f"("a.py":3:0) at "g"("b.py":7:1))))) -> tensor<4xf32> {
    %0 = stablehlo.negate %arg0 : tensor<4xf32> loc(#loc4)
    return %0 : tensor<4xf32> loc(#loc)
  } loc(#loc)
} loc(#loc)
#loc1 = loc("a.py":3:0)
#loc2 = loc("jit(f)/mul"(#loc1))
"""
    funcs = S.parse_module(text)
    assert [o.name for o in funcs["main"].ops] == ["multiply", "call", "return"]
    assert [o.name for o in funcs["inner"].ops] == ["negate", "return"]


# ---- the reference's own differentiation test inputs -------------------------------------------------------------

import json
import os

LIT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "lit_primal_functions.json")))

# Files of test/lit_tests/diffrules/stablehlo/ whose operators are on the llama path or next to it: every primal
# function in them must parse, print and parse again to the same operator list.
LIT_IN_SCOPE = ["add", "atan2", "broadcastindim", "broadcastindim2", "cbrt", "checked_mul", "clamp", "cosine", "divide",
                "dot_general_2", "dot_general_3", "dotgeneral_vectormode", "exponential", "exponential_minus_one",
                "gather", "log", "log_plus_one", "logistic", "maximum", "minimum", "negate", "pad", "power", "reduce",
                "reduceactivity", "rsqrt", "select", "sine", "sqrt", "subtract", "tanh", "transpose",
                "transpose_elem_batch_autodiff"]
# Files that hold a complex-valued variant next to the real one: the real functions must parse.
LIT_REAL_PART = ["abs", "dot_general", "multiply"]


@pytest.mark.parametrize("name", LIT_IN_SCOPE + LIT_REAL_PART)
def test_reference_lit_inputs_parse_and_print_to_a_fixed_point(name):
    from enzyme_ad.jax import stablehlo as H
    fns = LIT[name + ".mlir"]
    if name in LIT_REAL_PART:
        fns = [f for f in fns if "complex<" not in f]
    assert fns
    for fn in fns:
        m = H.parse_module("module {\n" + fn + "\n}")
        (f,) = m.values()
        assert f.ops and f.ops[-1].name == "return"
        again = H.parse_module(H.print_module(m))
        (g,) = again.values()
        assert [(o.name, len(o.operands), [repr(t) for t in o.types]) for o in f.ops] == \
               [(o.name, len(o.operands), [repr(t) for t in o.types]) for o in g.ops]


def test_reference_lit_inputs_out_of_scope_fail_cleanly():
    """Everything else in that directory (control flow, scatter, sort, convolution, FFT, complex numbers, dynamic
    slices, batch norm, einsum) is outside the llama path: the parser must say so by name, not crash."""
    from enzyme_ad.jax import stablehlo as H
    seen = 0
    for fname, fns in LIT.items():
        if fname[:-5] in LIT_IN_SCOPE + LIT_REAL_PART:
            continue
        for fn in fns:
            try:
                H.parse_module("module {\n" + fn + "\n}")
            except (NotImplementedError, H.ParseError) as e:
                assert str(e)
                seen += 1
    assert seen >= 30


def test_gather_rule_has_the_reference_ir_form():
    """gather.mlir: FORWARD = gather of the tangent table with the primal indices, next to the primal gather;
    REVERSE = one scatter-add of the cotangent rows into a zero table, here the emi_embedding_bwd target; the
    indices get no cotangent."""
    from enzyme_ad.jax import stablehlo as H, stablehlo_ad as AD
    (fn,) = LIT["gather.mlir"]
    f = H.parse_module("module {\n" + fn + "\n}")["main"]
    fwd = AD.forward_function(f, arg_active=[True, False])
    assert [o.name for o in fwd.ops] == ["gather", "gather", "return"]
    assert fwd.ops[0].operands[1] == fwd.ops[1].operands[1] and fwd.ops[1].operands[0].startswith("%t_")
    rev = AD.reverse_function(f, arg_active=[True, False])
    assert [o.name for o in rev.ops] == ["reshape", "custom_call", "return"]
    assert rev.ops[1].attrs["target"] == "emi_embedding_bwd" and repr(rev.result_types[0]) == "tensor<64x3xf32>"
    text = H.print_module({"main": rev})
    assert "@emi_embedding_bwd" in text and "api_version = 4" in text
    with pytest.raises(NotImplementedError):          # a gather that is not a row lookup is refused by name
        H.Executable  # noqa: B018  (the class exists)
        bad = fn.replace("slice_sizes = array<i64: 1, 3>", "slice_sizes = array<i64: 1, 2>")
        AD.reverse_function(H.parse_module("module {\n" + bad + "\n}")["main"], arg_active=[True, False])


# The mean softmax cross-entropy of integer targets in the form `jax.jit(f).lower(...).as_text()` prints for
#   f = lambda z, t: -jnp.mean(jnp.sum(jax.nn.one_hot(t, V) * jax.nn.log_softmax(z), axis=-1))
# (log_softmax: reduce max, subtract, exp, reduce add, log, subtract with keep-dims broadcasts; one_hot: targets
# spread along a new last axis compared with an iota over it).  Written by hand to that form: no JAX here.
def traced_cross_entropy_text(rows, V, dt="f32", select_form=False):
    lead = "x".join(str(r) for r in rows)
    R, n = len(rows), int(np.prod(rows))
    full, keep, flat = "tensor<%sx%dx%s>" % (lead, V, dt), "tensor<%sx1x%s>" % (lead, dt), "tensor<%sx%s>" % (lead, dt)
    ifull, ikeep, iflat = "tensor<%sx%dxi32>" % (lead, V), "tensor<%sx1xi32>" % lead, "tensor<%sxi32>" % lead
    iota = "tensor<%sx%dxi32>" % ("x".join("1" for _ in rows), V)
    d_flat, d_keep = list(range(R)), list(range(R + 1))
    onehot = ("%%15 = stablehlo.convert %%14 : (%s) -> %s\n      %%16 = stablehlo.multiply %%15, %%9 : %s" %
              (full.replace(dt + ">", "i1>"), full, full))
    if select_form:
        onehot = ("%%z = stablehlo.constant dense<0.000000e+00> : %s\n      %%16 = stablehlo.select %%14, %%9, %%z : %s, %s" %
                  (full, full.replace(dt + ">", "i1>"), full))
    return """
module @jit_loss {
  func.func public @main(%%arg0: %(full)s, %%arg1: %(iflat)s) -> (tensor<%(dt)s>) {
      %%cst = stablehlo.constant dense<%(ninf)s> : tensor<%(dt)s>
      %%0 = stablehlo.reduce(%%arg0 init: %%cst) applies stablehlo.maximum across dimensions = [%(R)d] : (%(full)s, tensor<%(dt)s>) -> %(flat)s
      %%1 = stablehlo.broadcast_in_dim %%0, dims = %(d_flat)s : (%(flat)s) -> %(keep)s
      %%2 = stablehlo.broadcast_in_dim %%1, dims = %(d_keep)s : (%(keep)s) -> %(full)s
      %%3 = stablehlo.subtract %%arg0, %%2 : %(full)s
      %%4 = stablehlo.exponential %%3 : %(full)s
      %%cst_0 = stablehlo.constant dense<0.000000e+00> : tensor<%(dt)s>
      %%5 = stablehlo.reduce(%%4 init: %%cst_0) applies stablehlo.add across dimensions = [%(R)d] : (%(full)s, tensor<%(dt)s>) -> %(flat)s
      %%6 = stablehlo.broadcast_in_dim %%5, dims = %(d_flat)s : (%(flat)s) -> %(keep)s
      %%7 = stablehlo.log %%6 : %(keep)s
      %%8 = stablehlo.broadcast_in_dim %%7, dims = %(d_keep)s : (%(keep)s) -> %(full)s
      %%9 = stablehlo.subtract %%3, %%8 : %(full)s
      %%10 = stablehlo.broadcast_in_dim %%arg1, dims = %(d_flat)s : (%(iflat)s) -> %(ikeep)s
      %%11 = stablehlo.iota dim = %(R)d : %(iota)s
      %%12 = stablehlo.broadcast_in_dim %%10, dims = %(d_keep)s : (%(ikeep)s) -> %(ifull)s
      %%13 = stablehlo.broadcast_in_dim %%11, dims = %(d_keep)s : (%(iota)s) -> %(ifull)s
      %%14 = stablehlo.compare  EQ, %%12, %%13,  SIGNED : (%(ifull)s, %(ifull)s) -> %(mask)s
      %(onehot)s
      %%17 = stablehlo.reduce(%%16 init: %%cst_0) applies stablehlo.add across dimensions = [%(R)d] : (%(full)s, tensor<%(dt)s>) -> %(flat)s
      %%18 = stablehlo.reduce(%%17 init: %%cst_0) applies stablehlo.add across dimensions = %(d_flat)s : (%(flat)s, tensor<%(dt)s>) -> tensor<%(dt)s>
      %%cst_1 = stablehlo.constant dense<%(n)d.0> : tensor<%(dt)s>
      %%19 = stablehlo.divide %%18, %%cst_1 : tensor<%(dt)s>
      %%20 = stablehlo.negate %%19 : tensor<%(dt)s>
      return %%20 : tensor<%(dt)s>
  }
}""" % dict(full=full, keep=keep, flat=flat, ifull=ifull, ikeep=ikeep, iflat=iflat, iota=iota, d_flat=d_flat, d_keep=d_keep, R=R,
           dt=dt, n=n, onehot=onehot, mask=full.replace(dt + ">", "i1>"), ninf="0xFF800000" if dt == "f32" else "0xFF80")


@pytest.mark.parametrize("rows,select_form", [((8,), False), ((2, 5), False), ((8,), True)])
def test_traced_cross_entropy_is_matched_and_lowered(rows, select_form):
    """The whole softmax / one-hot cluster becomes one emi.cross_entropy (printed as emi_cross_entropy_fwd); what is
    left is the mean.  Reverse mode calls emi_cross_entropy_bwd on the saved log-sum-exp with the targets inactive,
    forward mode emi_cross_entropy_jvp."""
    import enzyme_ad.jax as ej
    from enzyme_ad.jax import stablehlo as S
    from enzyme_ad.jax import stablehlo_ad as AD
    text = traced_cross_entropy_text(rows, 16, select_form=select_form)
    exe = S.Executable(text)
    assert exe.fused == {"cross_entropy": 1}
    names = [o.name for o in exe.funcs["main"].ops]
    for gone in ("exponential", "log", "compare", "iota", "convert", "select", "multiply", "subtract"):
        assert gone not in names, names
    ce = [o for o in exe.funcs["main"].ops if o.name == "emi.cross_entropy"][0]
    assert ce.operands == ["%arg0", "%arg1"] and ce.attrs == {"negated": True}
    n = int(np.prod(rows))
    low = ej.optimize_module(text)
    call = [l for l in low.splitlines() if "stablehlo.custom_call" in l]
    assert len(call) == 1 and "@emi_cross_entropy_fwd(" in call[0]
    assert ": (tensor<%dx16xf32>, tensor<%dxi32>) -> (tensor<%dxf32>, tensor<%dxf32>)" % (n, n, n, n) in call[0]
    assert S.print_module(S.parse_module(low)) == low
    rev = AD.reverse_module_text(text)
    rcalls = [l.split("@")[1].split("(")[0] for l in rev.splitlines() if "stablehlo.custom_call" in l]
    assert rcalls == ["emi_cross_entropy_fwd", "emi_cross_entropy_bwd"]
    bwd = [l for l in rev.splitlines() if "@emi_cross_entropy_bwd" in l][0]
    assert ": (tensor<%dx16xf32>, tensor<%dxi32>, tensor<%dxf32>, tensor<%dxf32>) -> tensor<%dx16xf32>" % (n, n, n, n, n) in bwd
    sig = S.parse_module(rev)["main"]
    assert [repr(t) for _, t in sig.args][-1] == "tensor<f32>" and len(sig.result_types) == 1        # d logits only
    fwd = AD.forward_module_text(text)
    assert [l.split("@")[1].split("(")[0] for l in fwd.splitlines() if "stablehlo.custom_call" in l] == \
        ["emi_cross_entropy_fwd", "emi_cross_entropy_jvp"]


def test_cross_entropy_cluster_is_left_alone_when_it_is_not_one():
    from enzyme_ad.jax import stablehlo as S
    text = traced_cross_entropy_text((8,), 16)
    # the log-probabilities are also returned: interior value used outside
    leaky = text.replace("-> (tensor<f32>)", "-> (tensor<f32>, tensor<8x16xf32>)").replace(
        "return %20 : tensor<f32>", "return %20, %9 : tensor<f32>, tensor<8x16xf32>")
    assert S.Executable(leaky).fused.get("cross_entropy", 0) == 0
    # compared with NE, or against an index that is not the class index: not a one-hot
    assert S.Executable(text.replace("compare  EQ", "compare  NE")).fused.get("cross_entropy", 0) == 0
    shifted = text.replace("%11 = stablehlo.iota dim = 1 : tensor<1x16xi32>",
                           "%11 = stablehlo.constant dense<[[1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16]]> : tensor<1x16xi32>")
    assert S.Executable(shifted).fused.get("cross_entropy", 0) == 0
    # the normaliser is the sum of exp of something else
    assert S.Executable(text.replace("%4 = stablehlo.exponential %3", "%4 = stablehlo.exponential %arg0")).fused.get("cross_entropy", 0) == 0
