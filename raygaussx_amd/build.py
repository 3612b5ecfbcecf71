"""Compiles librgx.so (HIP, gfx950) in-tree with hipcc.

``python -m raygaussx_amd.build`` or ``build()``.  The flags matter:
``-ffp-contract=off`` keeps the hit predicate's arithmetic identical to a CPU
evaluation (fused multiply-adds only where the source says fmaf);
``-munsafe-fp-atomics`` selects the hardware fp32 atomic add for the gradient
scatter; packed-fp32 code generation is disabled.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librgx.so")
SOURCES = ["rgx_api.hip", "rgx_build.hip", "rgx_pergauss.hip", "rgx_image.hip", "rgx_march.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
         "-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def build(verbose=False, extra=(), lib=LIB, tag=""):
    """``extra``: more hipcc flags; ``lib`` / ``tag``: write a differently named library and objects."""
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", tag + ".o"))
        cmd = ["hipcc", *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(out, file=sys.stderr)
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib]
    subprocess.check_call(cmd)
    return lib


if __name__ == "__main__":
    print(build(verbose=True))
