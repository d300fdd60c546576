"""Compiles the HIP extension (C-ABI shared library) for gfx950, in-tree.

    python -m megengine_amd.build

-ffp-contract=off and the correctly rounded divide are part of the arithmetic contract of the
epilogue; packed FP32 instructions are disabled for the device pass.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmi355_convbias.so")
SOURCES = ["capi.hip", "conv_direct.hip", "conv_igemm.hip", "conv_igemm_dma.hip", "conv_igemm2.hip", "conv_pw4.hip", "conv_c4.hip", "conv_dw.hip", "relayout.hip", "requant.hip", "pooling.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
]


def build(verbose=False, jobs=5):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = ["hipcc", *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _wait(procs)
    _wait(procs)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def _wait(procs):
    failed = []
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "not a recognized feature for this target" not in l)
        if p.returncode != 0:
            failed.append((src, out))
        elif out.strip():
            print(out)
    procs.clear()
    if failed:
        for src, out in failed:
            sys.stderr.write("---- %s ----\n%s\n" % (src, out))
        raise RuntimeError("hipcc failed for: %s" % ", ".join(s for s, _ in failed))


if __name__ == "__main__":
    print(build(verbose=True))
