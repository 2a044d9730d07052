"""The reference's fixtures written the way its own tests write them (a class per case with
`ins`, `dins`, `douts`, `fn`, `name` set in setUp; test/bench_vs_xla.py:5-52, test/testffi.py,
test/llama.py:241-319), run by the harness counterpart `enzyme_ad.jax.test_utils.EnzymeJaxTest`:
primal, forward mode and reverse mode under every pipeline, cross-checked and timed, rows in the
reference's columns."""
import csv
import os
import tempfile

import numpy as np
import pytest
import torch

from enzyme_ad.jax.test_utils import EnzymeJaxTest, no_newxla

pytestmark = pytest.mark.gpu


def arr(a):
    return torch.tensor(np.asarray(a, dtype=np.float32), device="cuda")


class _Case(EnzymeJaxTest):
    """Writes the CSV into a scratch directory and checks its shape after the run."""

    def test(self):
        if self.name is None:
            return
        with tempfile.TemporaryDirectory() as d:
            os.environ["TEST_UNDECLARED_OUTPUTS_DIR"] = d
            try:
                super().test()
                rows = list(csv.reader(open(os.path.join(d, "results_%s.csv" % self.__class__.__name__))))
            finally:
                del os.environ["TEST_UNDECLARED_OUTPUTS_DIR"]
        assert rows[0] == ["Benchmark Name", "Pass Pipeline", "Backend", "Key", "Time"]
        assert sorted(set(r[3] for r in rows[1:])) == ["BothRev", "Forward", "Primal"]
        assert set(r[1] for r in rows[1:]) == {"JaXPipe", "Jax", "IDefOpt"} and all(float(r[4]) > 0 for r in rows[1:])
        self.check()

    def check(self):
        pass


class AddOne(_Case):
    def setUp(self):
        from enzyme_ad.jax import ops
        self.ins = [arr([1.0, 2.0, 3.0]), arr([10.0, 20.0, 30.0])]
        self.dins = [arr([0.1, 0.2, 0.3]), arr([50.0, 70.0, 110.0])]
        self.douts = arr([500.0, 700.0, 110.0])

        def add_one(x, y):
            return ops.add(ops.add(x, torch.ones_like(x)), y)

        self.primfilter = self.fwdfilter = self.revfilter = no_newxla
        self.fn = add_one
        self.name = "add_one"

    def check(self):
        assert torch.equal(self.primres, arr([12.0, 23.0, 34.0]))
        assert torch.allclose(self.fwdres, arr([50.1, 70.2, 110.3]))
        assert all(torch.equal(g, self.douts) for g in self.revres)


class HLOFFI(_Case):
    def setUp(self):
        from enzyme_ad.jax import hlo_call
        from test_gpu_stablehlo import HLO_FFI

        def do_something(mat, scalar):
            a, b = hlo_call(mat, scalar, source=HLO_FFI)
            return a, b

        self.ins = [arr(np.ones((2, 2))), arr(2.7)]
        self.dins = [arr(np.full((2, 2), 5.0)), arr(3.1)]
        self.douts = (arr(3.4), arr(np.full((2, 2), 7.0)))
        self.fn = do_something
        self.name = "hlo_ffi"
        self.atol = 1e-4

    def check(self):
        assert float(self.primres[0]) == 4.0 and float(self.fwdres[0]) == 20.0
        assert abs(float(self.revres[1]) - 28.0) < 1e-4


class Llama(_Case):
    """test/llama.py:241-319: dim 288, hidden 768, 6 layers, 6 heads, uniform[0, 1) weights and
    input, zero caches of one row, compared with the reference's atol = rtol = 1e-3."""

    def setUp(self):
        from enzyme_ad.jax import llama
        cfg = {"dim": 288, "hidden_dim": 768, "n_layers": 6, "n_heads": 6, "n_kv_heads": 6, "vocab_size": 32000, "seq_len": 256}
        g = torch.Generator(device="cuda").manual_seed(0)
        u = lambda *shape: torch.rand(shape, device="cuda", generator=g)
        L, D, H = 6, 288, 768
        weights = {"rms_att_weight": u(L, D), "wq": u(L, D, D), "wk": u(L, D, D), "wv": u(L, D, D), "wo": u(L, D, D),
                   "rms_ffn_weight": u(L, D), "w1": u(L, H, D), "w2": u(L, D, H), "w3": u(L, H, D), "rms_final_weight": u(D)}
        x, dx = u(D), u(D)
        kc, vc = torch.zeros((L, 1, D), device="cuda"), torch.zeros((L, 1, D), device="cuda")
        self.fn = lambda x, weights, key_cache, value_cache: llama.forward_step(x, cfg, weights, key_cache, value_cache)
        self.name = "llama"
        self.ins = [x, weights, kc, vc]
        self.dins = [dx, {k: u(*v.shape) for k, v in weights.items()}, u(L, 1, D), u(L, 1, D)]
        self.douts = u(D)
        self.atol = self.rtol = 1e-3
        self.repeat = 3

    def check(self):
        assert self.primres.shape == (288,) and bool(torch.isfinite(self.primres).all())
        assert len(self.revres) == 4 and set(self.revres[1]) == set(self.ins[1])
