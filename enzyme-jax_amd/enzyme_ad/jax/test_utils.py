"""Counterpart of the reference's test harness (test/test_utils.py): a fixture class whose
subclasses set `ins`, `dins`, `douts`, `fn` and `name` in `setUp` (test/bench_vs_xla.py,
test/llama.py:241-319), and `harness`, which runs the primal, forward-mode and reverse-mode
programs under every pipeline, holds the results of all pipelines against the first one's with
`allclose(atol, rtol)` (`recursive_check`, :522-550), times them (`profile_compiled_function`)
and prints / writes rows in the reference's columns (:589-614):
    Benchmark Name, Pass Pipeline, Backend, Key, Time.
On this build every pipeline runs the same HIP kernels (the pass strings select nothing), so
the cross-pipeline check guards the host plumbing; keys are Primal, Forward and BothRev."""
import csv
import os
import unittest

import torch

from .primitives import JaXPipeline, enzyme_jax_ir, full_optimization_pass_pipeline, jvp, tree_flatten, vjp
from .profiling import CSV_HEADER, profile_compiled_function

AllBackends = ["rocm"]


def pipelines():
    """(name, pipeline options or None for the undecorated function, backends), the subset of
    test/test_utils.py:412-456 that differs in anything but optimizer pattern lists."""
    return [("JaXPipe", JaXPipeline(), AllBackends), ("Jax", None, AllBackends),
            ("IDefOpt", JaXPipeline(full_optimization_pass_pipeline()), AllBackends)]


def no_newxla(x):
    return x


def justjax(x):
    return [p for p in x if p[1] is None]


def splatjvp(in_fn):
    def fwd(*args):
        n = len(args) // 2
        return jvp(in_fn, tuple(args[:n]), tuple(args[n:]))
    return fwd


def splatvjp(in_fn):
    def rev(dout, *args):
        primals, f_vjp = vjp(in_fn, *args)
        return primals, f_vjp(dout)
    return rev


def splatvjp_noprim(in_fn):
    def rev(dout, *args):
        primals, f_vjp = vjp(in_fn, *args)
        return f_vjp(dout)
    return rev


def recursive_check(tester, lhs, rhs, pname=None):
    l1, d1 = tree_flatten(lhs)
    l2, d2 = tree_flatten(rhs)
    tester.assertEqual(len(l1), len(l2), "result trees differ (%s)" % pname)
    for a, b in zip(l1, l2):
        if not isinstance(a, torch.Tensor):
            tester.assertEqual(a, b)
            continue
        legal = bool(torch.allclose(a.float(), b.float(), atol=tester.atol, rtol=tester.rtol))
        if not legal:
            err = float((a.float() - b.float()).abs().max())
            if tester.skip_test_assert:
                print("Skipping test assert for %s %s but test failed with max error %g." % (tester.name, pname, err))
                continue
            print("lhs (%s)" % pname, a, "\nrhs", b, "\nmax", err)
        tester.assertTrue(legal, "%s: results differ" % pname)


class EnzymeJaxTest(unittest.TestCase):
    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.primfilter = lambda x: x
        self.fwdfilter = lambda x: x
        self.revfilter = lambda x: x
        self.repeat = 10
        self.AllBackends = AllBackends
        self.AllPipelines = pipelines()
        self.revprimal = True
        self.atol = 1e-6
        self.rtol = 0.0
        self.mlirad_fwd = True
        self.mlirad_rev = True
        self.results = []
        self.skip_test_assert = False

    def pretty_print_table(self, name, pname, backend, key, time):
        print("{:<20}\t{:<20}\t{:<15}\t{:<10}\t{:<15.8f}".format(name, pname, backend, key, time), flush=True)
        self.results.append("{}\t{}\t{}\t{}\t{}".format(name, pname, backend, key, time))

    def write_results_csv(self, filename=""):
        if filename == "":
            filename = "results_%s.csv" % self.__class__.__name__
        outfile = os.path.join(os.environ.get("TEST_UNDECLARED_OUTPUTS_DIR", "."), filename)
        with open(outfile, "w", newline="") as f:
            w = csv.writer(f)
            w.writerow(CSV_HEADER)
            for line in self.results:
                w.writerow(line.split("\t"))
        print("Results written to %s" % outfile)
        return outfile

    def setUp(self):
        self.name = None

    def test(self):
        if self.name is None:
            return
        self.harness(self.name, self.fn, self.ins, self.dins, self.douts)
        self.write_results_csv()

    def _wrap(self, in_fn, pipeline):
        return in_fn if pipeline is None else enzyme_jax_ir(pipeline_options=pipeline, inner_jit=False)(in_fn)

    def harness(self, name, in_fn, ins, dins, douts):
        if self.mlirad_fwd:
            assert len(ins) == len(dins)
        revtransform = splatvjp if self.revprimal else splatvjp_noprim
        for backend in self.AllBackends:
            primres = fwdres = revres = None
            for pname, pipeline, pbackends in self.primfilter(self.AllPipelines):
                if backend not in pbackends:
                    continue
                fn = self._wrap(in_fn, pipeline)
                ao = fn(*ins)
                if primres is None:
                    primres = ao
                else:
                    recursive_check(self, ao, primres, "Primal " + pname)
                self.pretty_print_table(name, pname, backend, "Primal", profile_compiled_function(fn, ins, nrepeat=self.repeat)[0])
            for pname, pipeline, pbackends in self.fwdfilter(self.AllPipelines):
                if backend not in pbackends or not (self.mlirad_fwd or pipeline is None):
                    continue
                fwd = splatjvp(self._wrap(in_fn, pipeline))
                all_ins = list(ins) + list(dins)
                primals, tangents = fwd(*all_ins)
                if primres is None:
                    primres = primals
                else:
                    recursive_check(self, primals, primres, "Primal " + pname)
                if fwdres is None:
                    fwdres = tangents
                else:
                    recursive_check(self, tangents, fwdres, "Forward " + pname)
                self.pretty_print_table(name, pname, backend, "Forward", profile_compiled_function(fwd, all_ins, nrepeat=self.repeat)[0])
            for pname, pipeline, pbackends in self.revfilter(self.AllPipelines):
                if backend not in pbackends or not (pipeline is None or (pipeline.mlir_ad() and self.mlirad_rev)):
                    continue
                rev = revtransform(self._wrap(in_fn, pipeline))
                all_ins = [douts] + list(ins)
                out = rev(*all_ins)
                if self.revprimal:
                    primals, grads = out
                    if primres is not None:
                        recursive_check(self, primals, primres, "Primal " + pname)
                else:
                    grads = out
                if revres is None:
                    revres = grads
                else:
                    recursive_check(self, grads, revres, "Reverse " + pname)
                self.pretty_print_table(name, pname, backend, "BothRev", profile_compiled_function(rev, all_ins, nrepeat=self.repeat)[0])
            self.primres, self.fwdres, self.revres = primres, fwdres, revres
