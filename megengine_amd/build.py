"""Compiles the HIP extension (C-ABI shared library) for gfx950, in-tree.

    python -m megengine_amd.build

-ffp-contract=off and the correctly rounded divide are part of the arithmetic contract of the
epilogue; packed FP32 instructions are disabled for the device pass.

The compiler's per-kernel resource report (-Rpass-analysis=kernel-resource-usage: registers, scratch bytes, waves per
SIMD) is collected into build/kernel_resources.json; tests/test_kernel_resources.py holds the hot kernels to their
budgets (a feature added behind a run-time flag once cost the fast kernels up to 77 VGPRs and 7 % of the benchmark).
"""
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmi355_convbias.so")
SOURCES = ["capi.hip", "conv_direct.hip", "conv_igemm.hip", "conv_igemm_dma.hip", "conv_igemm2.hip", "conv_igemm3.hip", "conv_igemm4.hip", "conv_pw4.hip", "conv_c4.hip", "conv_dw.hip", "conv_nchw.hip", "relayout.hip", "requant.hip", "elemwise_q.hip", "pooling.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
    "-Rpass-analysis=kernel-resource-usage",
]
RESOURCES = os.path.join(HERE, "build", "kernel_resources.json")


def build(verbose=False, jobs=5):
    objs = []
    procs = []
    _resources.clear()
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
    with open(RESOURCES, "w") as f:
        json.dump(_resources, f, indent=0, sort_keys=True)
    return LIB


_resources = {}
_FIELDS = {"VGPRs": "vgprs", "AGPRs": "agprs", "SGPRs": "sgprs", "ScratchSize [bytes/lane]": "scratch",
           "Occupancy [waves/SIMD]": "occupancy", "LDS Size [bytes/block]": "lds"}


def _demangle(names):
    try:
        out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True, check=True).stdout
        return out.splitlines()
    except Exception:
        return names


def _collect_resources(src, text):
    """Parses the resource remarks of one translation unit: {demangled kernel name: {vgprs, scratch, ...}}"""
    blocks = re.split(r"remark: [^\n]*Function Name: ", text)[1:]
    names = _demangle([b.split("\n")[0].split()[0] for b in blocks])
    for name, b in zip(names, blocks):
        entry = {"file": src}
        for key, short in _FIELDS.items():
            m = re.search(re.escape(key) + r": (\d+)", b)
            if m:
                entry[short] = int(m.group(1))
        _resources[name] = entry


def _without_remarks(text):
    """Compiler output minus the resource remarks (with their source snippets), the harmless warning about the
    packed-FP32 feature on the host pass and the closing counts."""
    keep, in_remark = [], False
    for l in text.splitlines():
        if re.search(r": (remark|warning|error|note):", l):
            in_remark = ": remark:" in l
        elif not re.match(r"^\s*(\d+)?\s*\|", l):
            in_remark = False
        if in_remark or "not a recognized feature for this target" in l or re.match(r"^\d+ (warning|remark)s? ", l) or " generated" in l and "remark" in l:
            continue
        keep.append(l)
    return "\n".join(keep)


def _wait(procs):
    failed = []
    for src, p in procs:
        out, _ = p.communicate()
        _collect_resources(src, out)
        out = _without_remarks(out)
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
