"""HIP-graph capture of a whole program of operator calls.

The reference compiles a decorated function once (`jax.jit`) and replays the executable; its
own benchmark case (test/llama.py: one token, dim 288) is a few hundred small kernels, so on a
GPU the step is bound by launch and host overhead, not by the kernels.  Here the counterpart of
the compiled executable is a captured HIP graph: `capture(fn, *example_args)` runs `fn` once
eagerly (so that trace-time constants such as RoPE tables and parsed-module constants exist),
records a second run into a graph on private memory, and returns a callable that copies new
argument values into the graph's input buffers and replays it.  `fn` may be any composition of
this package's operators, `vjp` / `jvp` / `hlo_call` included (e.g. `lambda *a: vjp(f, *a)[1](dy)`).

The result tensors belong to the graph and are overwritten by the next replay; clone what must
outlive it.  Argument shapes and dtypes are fixed at capture.  Nothing here records a memset
node: buffers are cleared by fill kernels.
"""
import torch

from .primitives import tree_flatten, tree_unflatten


class Captured:
    def __init__(self, fn, example_args):
        leaves, self._treedef = tree_flatten(tuple(example_args))
        for l in leaves:
            if isinstance(l, torch.Tensor) and not l.is_cuda:
                raise RuntimeError("argument is not in device memory: the HIP path has no CPU fallback")
        self._inputs = [l.clone() if isinstance(l, torch.Tensor) else l for l in leaves]
        args = tree_unflatten(self._treedef, self._inputs)
        side = torch.cuda.Stream()                       # default priority
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn(*args)                                    # eager run: fills caches, surfaces errors outside capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._outputs = fn(*args)
        self.replays = 0

    def __call__(self, *args):
        leaves, treedef = tree_flatten(tuple(args))
        if len(leaves) != len(self._inputs):
            raise ValueError("captured with %d argument leaves, called with %d" % (len(self._inputs), len(leaves)))
        for s, a in zip(self._inputs, leaves):
            if isinstance(s, torch.Tensor):
                if not isinstance(a, torch.Tensor) or a.shape != s.shape or a.dtype != s.dtype:
                    raise ValueError("argument does not match the captured %s/%s" % (tuple(s.shape), s.dtype))
                s.copy_(a)                               # device-to-device copy kernel on the current stream
            elif a != s:
                raise ValueError("non-tensor argument %r differs from the captured %r" % (a, s))
        self.graph.replay()
        self.replays += 1
        return self._outputs


def capture(fn, *example_args):
    """Capture `fn(*example_args)` into a HIP graph; the returned callable takes arguments of
    the same structure, shapes and dtypes and returns the graph's (reused) result tensors."""
    return Captured(fn, example_args)
