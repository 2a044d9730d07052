"""Builds libemi_hip.so (the gfx950 kernels + C ABI + XLA-FFI handlers) in-tree.

Usage: python enzyme-jax_amd/build.py [--force]
hipcc cross-compiles for gfx950 without a GPU; the resulting shared library
sits next to the sources so it travels with the tree.
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libemi_hip.so")
OBJDIR = os.path.join(LIBDIR, "obj")

HIP_SOURCES = ["elementwise.hip", "gemm.hip", "gemm_skinny.hip", "attention.hip", "attention_f32.hip", "attention_step.hip", "forward_mode.hip",
               "tensor_ops.hip", "cross_entropy.hip"]
CXX_SOURCES = ["status.cc", "ffi_handlers.cc"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-I", os.path.join(os.path.dirname(HERE), "include")]
# Packed-fp32 instruction selection is switched off for all device code.
HIP_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _digest(path):
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)) + ["../../include/emi.h"]:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    return h.hexdigest()


def build(force=False, verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    stamp = os.path.join(OBJDIR, "sources.sha256")
    digest = _digest(CSRC)
    if not force and os.path.exists(LIB) and os.path.exists(stamp) and open(stamp).read() == digest:
        return LIB
    jobs = []
    for s in HIP_SOURCES:
        obj = os.path.join(OBJDIR, s + ".o")
        jobs.append((obj, [HIPCC] + COMMON + HIP_FLAGS + ["-c", os.path.join(CSRC, s), "-o", obj]))
    for s in CXX_SOURCES:
        if not os.path.exists(os.path.join(CSRC, s)):
            continue
        obj = os.path.join(OBJDIR, s + ".o")
        jobs.append((obj, [HIPCC] + COMMON + ["-D__HIP_PLATFORM_AMD__", "-c", os.path.join(CSRC, s), "-o", obj]))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        outs = list(ex.map(lambda j: _run(j[1]), jobs))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + [j[0] for j in jobs])
    with open(stamp, "w") as f:
        f.write(digest)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
