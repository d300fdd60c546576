"""Parity at the benchmark workloads' full sizes, where the CPU checker cannot finish the whole tensor in seconds:
  * the checker evaluates the operator at tens of thousands of seeded random output positions;
  * the tiled kernel must agree with the generic direct kernel (checked against the checker on small
    shapes) on EVERY output element;
  * size-independent properties: an all-zero z changes nothing, RELU output is never negative and
    equals max(IDENTITY, 0) when the IDENTITY result did not saturate low.
These shapes make every persistent workgroup walk several tiles (incl. changing channel tiles)."""
import numpy as np
import pytest
import torch

from megengine_amd import _abi, lib, ops
from tests import util
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

DIRECT, IGEMM, DW, C4 = 0, 1, 2, 3


def dev_tensors(d, seed, bias_range=(-1000, 1000)):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    ss, fs, bs, ds = _abi.conv_shapes(d)
    src = torch.randint(-128, 128, ss, dtype=torch.int8, device="cuda", generator=g)
    flt = torch.randint(-127, 128, fs, dtype=torch.int8, device="cuda", generator=g)
    bias = torch.randint(int(bias_range[0]), int(bias_range[1]) + 1, bs, dtype=torch.int32, device="cuda", generator=g)
    z = torch.randint(-128, 128, ds, dtype=torch.int8, device="cuda", generator=g) if d.has_z else None
    return src, flt, bias, z


def spot_check(oracle, d, src, flt, bias, z, got, npoints=20000, seed=5):
    total = got.numel()
    idx = util.splitmix64(seed, npoints) % np.uint64(total)
    idx = idx.astype(np.int64)
    want = oracle.conv_bias_points(d, src.cpu().numpy(), flt.cpu().numpy(), bias.cpu().numpy(),
                                   None if z is None else z.cpu().numpy(), idx)
    g = got.reshape(-1)[torch.from_numpy(idx).cuda()].cpu().numpy()
    bad = np.nonzero(g != want)[0]
    assert len(bad) == 0, "%d / %d sampled outputs differ, first idx %d got %d want %d" % (
        len(bad), npoints, idx[bad[0]], g[bad[0]], want[bad[0]])


FULL_CASES = [
    # name, fmt, n, ic, hw, oc, f, stride, pad, nonline, z
    ("pw64_256", "NCHW32", 64, 64, 56, 256, 1, 1, 0, "RELU", True),        # config 1, expanding + z
    ("pw256_64", "NCHW32", 64, 256, 56, 64, 1, 1, 0, "IDENTITY", False),   # config 1
    ("pw2048_512", "NCHW32", 64, 2048, 7, 512, 1, 1, 0, "RELU", False),    # config 1
    ("r50_3x3", "NCHW32", 64, 128, 28, 128, 3, 1, 1, "RELU", False),       # config 2 body
    ("r50_3x3s2", "NCHW32", 64, 256, 28, 256, 3, 2, 1, "RELU", False),
    ("r50_ds", "NCHW32", 64, 256, 56, 512, 1, 2, 0, "IDENTITY", False),
    ("stem", "NCHW4", 16, 4, 224, 64, 7, 2, 3, "RELU", False),             # config 2 stem (batch 16)
    # first-layer kernel, eight tiles per workgroup (its ring of patch slots wraps twice), with a residual; and three
    # channel tiles of a 3x3 stem, so that a workgroup reloads its weights between tiles
    ("stem_bs64_z", "NCHW4", 64, 4, 224, 64, 7, 2, 3, "RELU", True),
    ("stem3x3_oc160", "NCHW4", 24, 4, 112, 160, 3, 1, 1, "H_SWISH", True),
    ("stem5x5s2_oc96", "NCHW4", 32, 4, 160, 96, 5, 2, 2, "IDENTITY", False),
    ("mbv2_expand", "NCHW4", 64, 24, 56, 144, 1, 1, 0, "RELU", False),     # config 3
    ("mbv2_project", "NCHW4", 64, 144, 56, 24, 1, 1, 0, "IDENTITY", True),
    # three / six channel tiles: successive tiles of a workgroup change channel tile, so the bias copy is rewritten
    ("oc384_3x3", "NCHW32", 16, 64, 56, 384, 3, 1, 1, "RELU", True),
    ("large_hswish", "NCHW32", 16, 256, 64, 256, 3, 1, 1, "H_SWISH", True),  # config 4a at batch 16
    ("large_5x5", "NCHW32", 8, 128, 80, 128, 5, 1, 2, "H_SWISH", True),      # config 4c at batch 8
]


@pytest.mark.parametrize("case", FULL_CASES, ids=[c[0] for c in FULL_CASES])
def test_igemm_full_size(oracle, case):
    name, fmt, n, ic, hw, oc, f, stride, pad, nl, z = case
    d = _abi.make_conv_desc(fmt, n, ic, hw, hw, oc, f, stride=stride, pad=pad, nonline=nl, has_z=z, scale_bias=2e-4,
                            scale_z=0.05, scale_dst=0.05)
    say("full-size", case)
    src, flt, bias, zt = dev_tensors(d, 17)
    algo, _ = ops.conv_bias_query(d)
    assert algo.id == (C4 if ic == 4 else IGEMM)   # 4-channel first layers have their own kernel
    got = ops.conv_bias_exec(d, src, flt, bias, zt, algo=algo)
    torch.cuda.synchronize()
    spot_check(oracle, d, src, flt, bias, zt, got)
    say("  heuristic", lib.algo_names()[algo.id], lib.tile_names()[algo.tile_cfg], "spot check ok; comparing with the direct kernel")
    ref = ops.conv_bias_exec(d, src, flt, bias, zt, algo=DIRECT)
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    # every tile configuration must give the same tensor
    for tile in range(len(lib.tile_names())):
        if not lib.tile_usable(d, tile):
            continue
        a2, _ = ops.conv_bias_query(d, IGEMM)
        a2.tile_cfg = tile
        say("  tile", lib.tile_names()[tile])
        out = ops.conv_bias_exec(d, src, flt, bias, zt, algo=a2)
        torch.cuda.synchronize()
        assert torch.equal(out, ref), lib.tile_names()[tile]
    if z:
        d0 = _abi.make_conv_desc(fmt, n, ic, hw, hw, oc, f, stride=stride, pad=pad, nonline=nl, has_z=False,
                                 scale_bias=2e-4, scale_dst=0.05)
        noz = ops.conv_bias_exec(d0, src, flt, bias, None)
        zero = ops.conv_bias_exec(d, src, flt, bias, torch.zeros_like(zt))
        torch.cuda.synchronize()
        assert torch.equal(noz, zero)


def live_scales(k, nonline):
    """Scales and a bias range that keep most outputs strictly inside the int8 range: uniform int8 operands give an
    accumulator of spread sigma = 73.9 * 73.3 * sqrt(K); the dst scale puts sigma at 25 output steps, the bias sits
    around +1.6 sigma (so that RELU keeps most values), the residual contributes at most +-32 steps."""
    sigma = 73.9 * 73.3 * k ** 0.5
    s_bias = 2e-4
    s_dst = float(np.float32(s_bias * sigma / 25.0))
    return dict(scale_bias=s_bias, scale_dst=s_dst, scale_z=0.25 * s_dst), (1.3 * sigma, 1.9 * sigma)


@pytest.mark.parametrize("case", FULL_CASES, ids=[c[0] for c in FULL_CASES])
def test_igemm_full_size_on_live_values(oracle, case):
    """The full-size cases again with scales derived from the reduction length: with the fixed 2e-4 / 0.05 pair a long
    reduction saturates most outputs, and a wrong accumulator in a few lanes would hide behind the clamp."""
    name, fmt, n, ic, hw, oc, f, stride, pad, nl, z = case
    scales, bias_range = live_scales(ic * f * f, nl)
    d = _abi.make_conv_desc(fmt, n, ic, hw, hw, oc, f, stride=stride, pad=pad, nonline=nl, has_z=z, **scales)
    say("full-size live", case, scales)
    src, flt, bias, zt = dev_tensors(d, 19, bias_range)
    ref = ops.conv_bias_exec(d, src, flt, bias, zt, algo=DIRECT)
    torch.cuda.synchronize()
    lo = 0 if nl == "RELU" else -128
    live = float(((ref > lo) & (ref < 127)).float().mean())
    say("  live outputs %.3f" % live)
    assert live >= 0.75
    spot_check(oracle, d, src, flt, bias, zt, ref)
    algo, _ = ops.conv_bias_query(d)
    got = ops.conv_bias_exec(d, src, flt, bias, zt, algo=algo)
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    if algo.id != IGEMM:
        return
    for tile in range(len(lib.tile_names())):
        if not lib.tile_usable(d, tile):
            continue
        a2, _ = ops.conv_bias_query(d, IGEMM)
        a2.tile_cfg = tile
        say("  tile", lib.tile_names()[tile])
        out = ops.conv_bias_exec(d, src, flt, bias, zt, algo=a2)
        torch.cuda.synchronize()
        assert torch.equal(out, ref), lib.tile_names()[tile]


def test_relu_property_full_size():
    d_id = _abi.make_conv_desc("NCHW32", 64, 64, 56, 56, 64, 3, pad=1, nonline="IDENTITY", scale_bias=2e-4, scale_dst=0.05)
    d_re = _abi.make_conv_desc("NCHW32", 64, 64, 56, 56, 64, 3, pad=1, nonline="RELU", scale_bias=2e-4, scale_dst=0.05)
    src, flt, bias, _ = dev_tensors(d_id, 3)
    a = ops.conv_bias_exec(d_id, src, flt, bias, None)
    b = ops.conv_bias_exec(d_re, src, flt, bias, None)
    torch.cuda.synchronize()
    assert int(b.min()) >= 0
    assert torch.equal(b, torch.clamp(a, min=0))


def test_depthwise_full_size(oracle):
    """config 3 depthwise layers: spot check + agreement with the direct kernel."""
    for (c, hw, stride) in ((96, 112, 2), (144, 56, 1), (960, 7, 1)):
        d = _abi.make_conv_desc("NCHW4", 64, c, hw, hw, c, 3, group=c, stride=stride, pad=1, nonline="RELU",
                                scale_bias=2e-4, scale_dst=0.05)
        say("depthwise full-size", c, hw, stride)
        src, flt, bias, _ = dev_tensors(d, 23)
        algo, _ = ops.conv_bias_query(d)
        assert algo.id == DW
        got = ops.conv_bias_exec(d, src, flt, bias, None, algo=algo)
        torch.cuda.synchronize()
        spot_check(oracle, d, src, flt, bias, None, got, npoints=20000)
        ref = ops.conv_bias_exec(d, src, flt, bias, None, algo=DIRECT)
        torch.cuda.synchronize()
        assert torch.equal(got, ref)
        # the same layer on live values (9 taps: sigma = 16 250; a bias around +1.6 sigma keeps RELU from zeroing half)
        scales, bias_range = live_scales(9, "RELU")
        d = _abi.make_conv_desc("NCHW4", 64, c, hw, hw, c, 3, group=c, stride=stride, pad=1, nonline="RELU", **scales)
        src, flt, bias, _ = dev_tensors(d, 29, bias_range)
        got = ops.conv_bias_exec(d, src, flt, bias, None, algo=algo)
        ref = ops.conv_bias_exec(d, src, flt, bias, None, algo=DIRECT)
        torch.cuda.synchronize()
        live = float(((ref > 0) & (ref < 127)).float().mean())
        say("  live outputs %.3f" % live)
        assert live >= 0.75
        spot_check(oracle, d, src, flt, bias, None, got, npoints=20000)
        assert torch.equal(got, ref)
