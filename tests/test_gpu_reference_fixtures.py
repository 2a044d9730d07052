"""The reference's small closed-form differentiation cases (test/bench_vs_xla.py:5-194) run through
`jvp` and `vjp` on the GPU and compared with answers worked out by hand from the inputs the
reference's fixtures hold: AddTwo, ActivityMismatch, GenDot and Concat written with the
operators of the transformer path, Sum, Cache and Slicing (which need reductions, broadcasts
and elementwise products) as StableHLO text through `hlo_call`."""
import numpy as np
import pytest
import torch

from gpu_util import host

pytestmark = pytest.mark.gpu


def f32(a):
    return torch.tensor(np.asarray(a, dtype=np.float32), device="cuda")


def sq(lo, hi):
    return sum(i * i for i in range(lo, hi))


def test_add_two_inactive_argument():
    """AddTwo (bench_vs_xla.py:32-52): f(x, z, y) = x + y; z gets a zero cotangent."""
    from enzyme_ad.jax import enzyme_jax_ir, jvp, vjp, ops

    @enzyme_jax_ir()
    def add_two(x, z, y):
        return ops.add(x, y)

    ins = [f32([1, 2, 3]), f32([10, 20, 30]), f32([100, 200, 300])]
    dins = [f32([0.1, 0.2, 0.3]), f32([50, 70, 110]), f32([1300, 1700, 1900])]
    out, tan = jvp(add_two, ins, dins)
    assert torch.equal(out, f32([101, 202, 303]))
    np.testing.assert_allclose(host(tan), [1300.1, 1700.2, 1900.3], rtol=1e-7)
    out, f_vjp = vjp(add_two, *ins)
    gx, gz, gy = f_vjp(f32([500, 700, 110]))
    assert torch.equal(gx, f32([500, 700, 110])) and torch.equal(gy, gx)
    assert torch.equal(gz, torch.zeros_like(gz))
    # the pipeline the reference would run for this reverse pass (primitives.py:1385-1419)
    assert ("retTys=enzyme_active argTys=enzyme_active,enzyme_active,enzyme_active mode=ReverseModeCombined"
            in add_two.last_pipeline.pass_pipeline())


def test_activity_mismatch():
    """ActivityMismatch (bench_vs_xla.py:111-134): a constant row with an active row
    appended; k = ones(12, 12) . x."""
    from enzyme_ad.jax import enzyme_jax_ir, jvp, vjp, ops

    dim = 12

    @enzyme_jax_ir()
    def f(x):
        k = ops.matmul_nt(x, torch.ones(dim, dim, device="cuda"))
        return ops.append_row(torch.zeros(1, dim, device="cuda"), k)

    x = f32(range(dim))
    dx = f32([i * i for i in range(dim)])
    out, tan = jvp(f, (x,), (dx,))
    assert out.shape == (2, dim)
    assert torch.equal(out, f32([[0.0] * dim, [66.0] * dim]))
    assert torch.equal(tan, f32([[0.0] * dim, [float(sq(0, dim))] * dim]))            # 506
    out, f_vjp = vjp(f, x)
    (gx,) = f_vjp(f32([i * i for i in range(2 * dim)]).reshape(2, dim))
    assert torch.equal(gx, f32([float(sq(dim, 2 * dim))] * dim))                      # 3818


def test_gen_dot():
    """GenDot (bench_vs_xla.py:137-168): ones(12,12) . x, then a batched product with
    ones(2,6,6) over the two halves, appended to a constant row."""
    from enzyme_ad.jax import enzyme_jax_ir, jvp, vjp, ops

    dim = 12
    h = dim // 2

    @enzyme_jax_ir()
    def f(x):
        k = ops.matmul_nt(x, torch.ones(dim, dim, device="cuda"))
        k_tmp = ops.reshape(k, (2, h))
        toconv2 = torch.ones(2, h, h, device="cuda")
        rows = [ops.matmul_nt(ops.select(k_tmp, i), toconv2[i]) for i in range(2)]
        k = ops.reshape(ops.append_row(ops.reshape(rows[0], (1, h)), rows[1]), (dim,))
        return ops.append_row(torch.zeros(1, dim, device="cuda"), k)

    x = f32(range(dim))
    dx = f32([i * i for i in range(dim)])
    out, tan = jvp(f, (x,), (dx,))
    assert torch.equal(out, f32([[0.0] * dim, [6.0 * 66.0] * dim]))
    assert torch.equal(tan, f32([[0.0] * dim, [6.0 * sq(0, dim)] * dim]))             # 3036
    out, f_vjp = vjp(f, x)
    (gx,) = f_vjp(f32([i * i for i in range(2 * dim)]).reshape(2, dim))
    # d k_tmp[i, :] = sum of the cotangent over half i; dx = ones^T . dk = 6 (both halves)
    assert torch.equal(gx, f32([6.0 * sq(dim, 2 * dim)] * dim))                        # 22908


def test_concat():
    """Concat (bench_vs_xla.py:171-194): two vectors joined; each cotangent is its slice."""
    from enzyme_ad.jax import enzyme_jax_ir, jvp, vjp, ops

    dim = 12

    @enzyme_jax_ir()
    def f(x, y):
        return ops.reshape(ops.append_row(ops.reshape(x, (1, dim)), y), (2 * dim,))

    x, y = f32(range(dim)), f32([10 * i for i in range(dim)])
    dx, dy = f32([i * i for i in range(dim)]), f32([i * i * i / 3.0 for i in range(dim)])
    out, tan = jvp(f, (x, y), (dx, dy))
    assert torch.equal(out, torch.cat([x, y])) and torch.equal(tan, torch.cat([dx, dy]))
    out, f_vjp = vjp(f, x, y)
    c = f32([i * i for i in range(2 * dim)])
    gx, gy = f_vjp(c)
    assert torch.equal(gx, c[:dim]) and torch.equal(gy, c[dim:])


def _text_case(text, ins, dins, douts):
    from enzyme_ad.jax import hlo_call, jvp, vjp

    fn = lambda *a: hlo_call(*a, source=text)[0]
    out, tan = jvp(fn, tuple(ins), tuple(dins))
    _, f_vjp = vjp(fn, *ins)
    return out, tan, f_vjp(douts)


def test_sum():
    """Sum (bench_vs_xla.py:55-69): jnp.sum over range(50)."""
    text = """func.func @main(%x: tensor<50xf32>) -> tensor<f32> {
      %z = stablehlo.constant dense<0.000000e+00> : tensor<f32>
      %r = stablehlo.reduce(%x init: %z) applies stablehlo.add across dimensions = [0] : (tensor<50xf32>, tensor<f32>) -> tensor<f32>
      return %r : tensor<f32>
    }"""
    out, tan, (gx,) = _text_case(text, [f32(range(50))], [f32([i * i for i in range(50)])], f32(1.0))
    assert float(out) == 1225.0 and float(tan) == float(sq(0, 50))                    # 40425
    assert torch.equal(gx, f32([1.0] * 50))


def test_cache():
    """Cache (bench_vs_xla.py:72-91): x * x[0] with x = range(288): x[0] = 0, so the output and
    the tangent vanish and the whole cotangent lands on x[0]: sum_j dout_j x_j = sum j^3."""
    dim = 288
    text = """func.func @main(%x: tensor<288xf32>) -> tensor<288xf32> {
      %s = stablehlo.slice %x [0:1] : (tensor<288xf32>) -> tensor<1xf32>
      %h = stablehlo.reshape %s : (tensor<1xf32>) -> tensor<f32>
      %b = stablehlo.broadcast_in_dim %h, dims = [] : (tensor<f32>) -> tensor<288xf32>
      %r = stablehlo.multiply %x, %b : tensor<288xf32>
      return %r : tensor<288xf32>
    }"""
    sqs = f32([i * i for i in range(dim)])
    out, tan, (gx,) = _text_case(text, [f32(range(dim))], [sqs], sqs)
    assert torch.equal(out, torch.zeros_like(out)) and torch.equal(tan, torch.zeros_like(tan))
    want = np.zeros(dim)
    want[0] = float(sum(j ** 3 for j in range(dim)))                                  # 1708003584
    np.testing.assert_allclose(host(gx), want, rtol=1e-5)                             # the reference's own rtol (:90)


def test_slicing():
    """Slicing (bench_vs_xla.py:94-108): x[0, 0:1, 0] * ones(3) on x = range(3) shaped (1, 3, 1)."""
    text = """func.func @main(%x: tensor<1x3x1xf32>) -> tensor<3xf32> {
      %s = stablehlo.slice %x [0:1, 0:1, 0:1] : (tensor<1x3x1xf32>) -> tensor<1x1x1xf32>
      %h = stablehlo.reshape %s : (tensor<1x1x1xf32>) -> tensor<1xf32>
      %one = stablehlo.constant dense<1.000000e+00> : tensor<3xf32>
      %b = stablehlo.broadcast_in_dim %h, dims = [0] : (tensor<1xf32>) -> tensor<3xf32>
      %r = stablehlo.multiply %b, %one : tensor<3xf32>
      return %r : tensor<3xf32>
    }"""
    x = f32(range(3)).reshape(1, 3, 1)
    out, tan, (gx,) = _text_case(text, [x], [f32([0.0, 1.0, 4.0]).reshape(1, 3, 1)], f32([0.0, 1.0, 4.0]))
    assert torch.equal(out, f32([0.0] * 3)) and torch.equal(tan, f32([0.0] * 3))
    assert torch.equal(gx, f32([5.0, 0.0, 0.0]).reshape(1, 3, 1))
