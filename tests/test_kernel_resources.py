"""Register and scratch budgets of the hot kernels, from the compiler's own resource report collected at build time
(megengine_amd/build/kernel_resources.json, written by megengine_amd.build).  These kernels are tuned around their
occupancy: a change that makes the fast-epilogue instantiations carry the registers of a rarely used path (it happened:
+10..77 VGPRs, spills on the 256-wide tiles, 7 % of the benchmark) must fail here, on the CPU, before it reaches a GPU."""
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PATH = os.path.join(ROOT, "megengine_amd", "build", "kernel_resources.json")


@pytest.fixture(scope="module")
def resources():
    if not os.path.exists(PATH):
        pytest.skip("no resource report: the library was not built in this tree")
    with open(PATH) as f:
        return json.load(f)


def kernels(resources, pattern):
    rx = re.compile(pattern)
    found = {k: v for k, v in resources.items() if rx.search(k)}
    assert found, "no kernel matches %s" % pattern
    return found


# second-generation kernel, fast epilogue (last template argument false):
#   igemm2_kernel<out pack, BM, BN, wave rows, wave cols, k chunks, ring, waves/SIMD bound, pointwise, K tail, general,
#                 wave groups that split the reduction (1 here)>
V2_BUDGETS = [
    # tile                       VGPRs  scratch  waves/SIMD
    (r"64, 128, 2, 2, \d, \d, 2", 112, 0, 4),     # 64x128 tiles (two workgroups per CU by LDS)
    (r"128, 64, 2, 2, \d, \d, 2", 112, 0, 4),
    (r"64, 64, 2, 2, 4, \d, 3", 84, 0, 6),        # 64x64: three workgroups per CU
    (r"128, 128, 2, 2, 2, \d, 2", 168, 0, 3),     # 128x128x64, four waves
    (r"128, 128, 2, 4, 2, 4, 4", 128, 0, 4),      # 128x128x64, eight waves
    (r"256, 128, 4, 2, 2, 3, 4", 128, None, 4),   # 8-wave tiles of 256: bound to four waves per SIMD
    (r"128, 256, 2, 4, 2, 3, 4", 128, None, 4),
    (r"256, 256, 4, 2, 2, 3, 2", 256, 0, 2),
]


@pytest.mark.parametrize("tile,vgprs,scratch,occupancy", V2_BUDGETS)
def test_second_generation_fast_kernels_keep_their_budget(resources, tile, vgprs, scratch, occupancy):
    ks = kernels(resources, r"igemm2_kernel<(32|4), %s, (true|false), (true|false), false, 1>" % tile)
    for name, r in ks.items():
        assert r["vgprs"] <= vgprs, (name, r)
        assert r["occupancy"] >= occupancy, (name, r)
        if scratch is not None:
            assert r["scratch"] <= scratch, (name, r)


def test_large_tiles_spill_little(resources):
    """The 256 x 128 / 128 x 256 tiles are compiled for four waves per SIMD (128 VGPRs): a few spilled dwords are the price
    of two workgroups per CU; more than that means something joined their register set."""
    for name, r in kernels(resources, r"igemm2_kernel<32, (256, 128, 4, 2|128, 256, 2, 4), 2, 3, 4, (true|false), (true|false), false, 1>").items():
        assert r["scratch"] <= 64, (name, r)


def test_first_generation_kernels_do_not_spill(resources):
    # igemm_dma_kernel<out pack, BM, BN, wave rows, wave cols, k chunks, ring, waves/SIMD bound, pointwise, in pack>
    # (two table-path variants compiled for four and six waves per SIMD keep 2-4 spilled dwords; the six-waves-per-SIMD
    # pointwise tile keeps one or two, stored and reloaded once per tile, outside the k-loop)
    for name, r in kernels(resources, r"igemm_dma_kernel<32, \d+, \d+, \d, \d, \d, \d, \d, (true|false), 32>").items():
        assert r["scratch"] <= (16 if ", false, 32>" in name else 8 if ", 6, true, 32>" in name else 0), (name, r)
    # the tile of the residual layers: three workgroups of eight waves per CU
    for name, r in kernels(resources, r"igemm_dma_kernel<32, 128, 128, 2, 4, 2, 3, 6, true, 32>").items():
        assert r["occupancy"] >= 6 and r["vgprs"] <= 80, (name, r)


def test_general_epilogue_lives_in_its_own_instantiations(resources):
    gen = kernels(resources, r"igemm2_kernel<(32|4), [^>]*, true, 1>")
    tiles = {re.search(r"igemm2_kernel<(?:32|4), (\d+, \d+), ", k).group(1) for k in gen}
    assert tiles == {"128, 128", "64, 128"}, tiles


def test_patch_staged_kernels_use_no_scratch(resources):
    """igemm3_kernel: a selection among per-lane values by a run-time index was once folded into an indexed load from
    scratch memory, and a scratch load in a loop that keeps LDS-direct copies in flight is followed by vmcnt(0): it
    empties the ring.  (The kernels keep such values in scalars selected by compares.)"""
    for name, r in kernels(resources, r"igemm3_kernel<").items():
        assert r["scratch"] == 0, (name, r)


def test_second_generation_kernels_use_no_scratch_in_the_tiles_the_heuristic_takes(resources):
    for name, r in kernels(resources, r"igemm2_kernel<(32|4), (128, 128, 2, 2, 2, 4|64, 128, 2, 2, 4, 3|64, 128, 2, 2, 2, 4|64, 64, 2, 2, 4, 4), \d, (true|false), (true|false), false, 1>").items():
        assert r["scratch"] == 0, (name, r)


def test_ring_kernels_with_register_resident_weights_use_no_scratch(resources):
    """c4_kernel and igemm4_kernel keep their weights in registers across a tile loop that has LDS-direct copies in
    flight: a spill there is reloaded with vmcnt(0) inside the loop and empties the ring.  The first-layer kernel for the
    7x7 stem must also leave room for four workgroups per CU."""
    c4 = kernels(resources, r"c4_kernel<")
    r4 = kernels(resources, r"igemm4_kernel<")
    assert len(c4) == 12 and len(r4) == 4
    for name, r in list(c4.items()) + list(r4.items()):
        assert r["scratch"] == 0, (name, r)
    for name, r in kernels(resources, r"c4_kernel<2, false, 7>").items():
        assert r["vgprs"] <= 128, (name, r)


def test_streaming_pointwise_kernels_keep_accumulators_in_vgprs(resources):
    """pw32s_kernel is bound by its vector instructions: accumulators in AGPRs would cost a move in and a move out per
    output (the compiler picks the VGPR form of the MFMA only when the launch bounds cap the register file at 256), and
    three workgroups per CU must fit.  Its only LDS is the kilobyte of the residual table (variants with a residual)."""
    ks = kernels(resources, r"pw32s_kernel<")
    assert len(ks) == 16
    for name, r in ks.items():
        assert r["agprs"] == 0 and r["scratch"] == 0, (name, r)
        assert r["lds"] <= (1024 if ", true>" in name else 16), (name, r)
        assert r["occupancy"] >= 3, (name, r)
