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
    with pytest.raises(NotImplementedError, match="stablehlo.cbrt"):
        S.parse_module("func.func @main(%a: tensor<f32>) -> tensor<f32> {\n %b = stablehlo.cbrt %a : tensor<f32>\n return %b : tensor<f32>\n}")
    with pytest.raises(S.ParseError):
        S.parse_module("func.func @main(%a: tensor<?xf32>) -> tensor<2xf32> {\n return %a : tensor<2xf32>\n}")
    with pytest.raises(S.ParseError):
        S.parse_module("module {}")


def test_llama_text_clusters_are_matched():
    from enzyme_ad.jax import stablehlo as S

    text, order = llama_step_text(CFG, pos=3)
    exe = S.Executable(text)
    L = CFG["n_layers"]
    assert exe.fused == {"rmsnorm": 2 * L + 1, "swiglu": L, "rope": 2 * L, "softmax_dot": 6 * L, "attention_step": L}
    left = Counter(o.name for o in exe.funcs["main"].ops)
    # what stays generic: weight slices / reshapes, the seven projections per layer, the two
    # cache appends per layer, the two residual adds per layer
    assert left["dot_general"] == 7 * L and left["concatenate"] == 2 * L and left["add"] == 2 * L
    assert not any(k in left for k in ("exponential", "reduce", "sqrt", "divide", "multiply", "broadcast_in_dim", "constant"))
    att = [o for o in exe.funcs["main"].ops if o.name == "emi.attention_step"][0]
    assert att.attrs["heads"] == 6 and att.attrs["rows"] == 4 and abs(att.attrs["scale"] - 1 / np.sqrt(48)) < 1e-7
    rope = [o for o in exe.funcs["main"].ops if o.name == "emi.rope"][0]
    assert rope.attrs["table"].shape == (144, 2)
    # unfused: only the constant folder ran (sqrt of the head size became a constant)
    plain = S.Executable(text, fuse=False)
    names = Counter(o.name for o in plain.funcs["main"].ops)
    assert plain.fused == {} and names["sqrt"] == 2 * L + 1 and names["exponential"] == 7 * L


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
    assert S.Executable(text).fused["swiglu"] == 0
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
    assert S.Executable(bad).fused["rope"] == 0


def test_optimize_module_prints_typed_ffi_custom_calls():
    """optimize_module: clusters come back as stablehlo.custom_call @emi_* in the typed-FFI wire
    format (api_version 4, scalars in backend_config, row-major layouts); the printed module
    parses again and printing it once more changes nothing."""
    import enzyme_ad.jax as ej
    from enzyme_ad.jax import stablehlo as S

    text, order = llama_step_text(dict(CFG, n_layers=1), pos=3)
    low = ej.optimize_module(text)
    calls = [l.strip() for l in low.splitlines() if "stablehlo.custom_call" in l]
    assert Counter(l.split("@")[1].split("(")[0] for l in calls) == {"emi_rmsnorm_fwd": 3, "emi_rope": 2, "emi_attn_step_fwd": 1, "emi_swiglu_fwd": 1}
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
