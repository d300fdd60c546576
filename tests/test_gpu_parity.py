"""Parity of the HIP kernels (through the C ABI) against the CPU checker: bit-exact int8.
Every case prints what it is about to launch before touching the GPU."""
import numpy as np
import pytest
import torch

from megengine_amd import _abi, lib, ops
from tests import util
from tests.gpu_util import check_case, run_gpu, say, to_dev

pytestmark = pytest.mark.gpu

DIRECT, IGEMM, DW, C4 = 0, 1, 2, 3
S = dict(scale_bias=2e-4, scale_z=0.05, scale_dst=0.05)


# ---------------------------------------------------------------------------------------------
# generic direct kernel: every format / mode on small shapes
# ---------------------------------------------------------------------------------------------

DIRECT_CASES = [
    dict(fmt="NCHW", n=2, ic=3, ih=7, iw=9, oc=5, fh=3, pad=1),
    dict(fmt="NCHW", n=1, ic=8, ih=8, iw=8, oc=12, fh=3, fw=2, group=4, pad=(1, 0), stride=(2, 1)),
    dict(fmt="NCHW", n=2, ic=4, ih=11, iw=10, oc=6, fh=3, group=2, pad=2, stride=(1, 2), dilate=2),
    dict(fmt="NCHW", n=1, ic=3, ih=8, iw=8, oc=4, fh=3, pad=1, mode=_abi.MODE_CONVOLUTION),
    dict(fmt="NCHW", n=1, ic=6, ih=9, iw=9, oc=6, fh=5, group=6, pad=2),
    dict(fmt="NCHW4", n=2, ic=8, ih=6, iw=5, oc=12, fh=3, pad=1),
    dict(fmt="NCHW4", n=1, ic=60, ih=9, iw=9, oc=20, fh=3, group=5, pad=1),   # shape family of naive/convolution.cpp:215
    dict(fmt="NCHW4", n=2, ic=16, ih=7, iw=7, oc=16, fh=3, group=16, pad=1),  # packed channel-wise
    dict(fmt="NCHW32", n=2, ic=32, ih=4, iw=4, oc=32, fh=3, pad=1),           # naive/conv_bias.cpp:163
    dict(fmt="NCHW32", n=1, ic=64, ih=5, iw=6, oc=64, fh=1, group=2),
    dict(fmt="NCHW44", n=1, ic=8, ih=5, iw=5, oc=8, fh=3, pad=1),
    dict(fmt="NCHW44", n=1, ic=16, ih=5, iw=5, oc=8, fh=3, group=2, pad=1),
    dict(fmt="NCHW44", n=1, ic=8, ih=6, iw=6, oc=8, fh=3, group=8, pad=1, stride=2),
    dict(fmt="NCHW4_NCHW32", n=1, ic=8, ih=6, iw=6, oc=32, fh=3, pad=1),
    dict(fmt="NCHW32_NCHW4", n=1, ic=32, ih=6, iw=6, oc=8, fh=3, pad=1),
]


def mk(c, **extra):
    kw = dict(c)
    kw.update(extra)
    fmt = kw.pop("fmt")
    return _abi.make_conv_desc(fmt, kw.pop("n"), kw.pop("ic"), kw.pop("ih"), kw.pop("iw"), kw.pop("oc"),
                               kw.pop("fh"), kw.pop("fw", None), **kw)


@pytest.mark.parametrize("i", range(len(DIRECT_CASES)))
def test_direct_all_formats(oracle, i):
    c = DIRECT_CASES[i]
    mixed = c["fmt"] in ("NCHW4_NCHW32", "NCHW32_NCHW4")
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in ((False,) if mixed else (False, True)):
            check_case(oracle, mk(c, nonline=nl, has_z=has_z, **S), seed=i + 1, algo=DIRECT, tag="direct%d" % i)


NCHW4_NCHW_CASES = [
    # shape family of the reference's own test of the format (dnn/test/cuda/conv_bias_int8.cpp:917-958), reduced
    dict(fmt="NCHW4_NCHW", n=2, ic=16, ih=23, iw=20, oc=20, fh=3, pad=1),
    dict(fmt="NCHW4_NCHW", n=2, ic=16, ih=12, iw=16, oc=24, fh=3, pad=1, stride=2),
    dict(fmt="NCHW4_NCHW", n=1, ic=16, ih=9, iw=10, oc=4, fh=3),
    dict(fmt="NCHW4_NCHW", n=2, ic=24, ih=8, iw=8, oc=6, fh=3, group=2, pad=1),
]


@pytest.mark.parametrize("i", range(len(NCHW4_NCHW_CASES)))
def test_nchw4_nchw(oracle, i):
    """NCHW4 activations and filter, NCHW dst: quantized dst bit-exact, Float32 dst to the reference checker's tolerance
    and exactly where float arithmetic is exact (unit scales, small integers)."""
    c = NCHW4_NCHW_CASES[i]
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            check_case(oracle, mk(c, nonline=nl, has_z=has_z, **S), seed=40 + i, algo=DIRECT, tag="nchw4_nchw s8")
            check_case(oracle, mk(c, nonline=nl, has_z=has_z, dst_dtype=_abi.DT_F32, scale_bias=1.9980618, scale_z=1.9980927),
                       seed=50 + i, tag="nchw4_nchw f32", src_range=(-3, 3), flt_range=(-3, 3), bias_range=(-200, 200),
                       z_range=(-128, 127))
            check_case(oracle, mk(c, nonline=nl, has_z=has_z, dst_dtype=_abi.DT_F32, scale_bias=0.0173, scale_z=0.0041),
                       seed=60 + i, tag="nchw4_nchw f32 full range")
    # exact: unit scales, so every float product and partial sum is a small integer
    d = mk(c, nonline="RELU", has_z=True, dst_dtype=_abi.DT_F32, scale_bias=1.0, scale_z=0.5)
    src, flt, bias, z = util.make_tensors(d, seed=70 + i, src_range=(-8, 8), flt_range=(-8, 8))
    want = oracle.conv_bias(d, src, flt, bias, z)
    got = run_gpu(d, src, flt, bias, z)
    assert np.array_equal(got, want)
    check_case(oracle, mk(c, dst_dtype=_abi.DT_QS32, scale_bias=2e-4, scale_dst=2e-4), seed=80 + i, algo=DIRECT,
               tag="nchw4_nchw s32")


NCHW4_NCHW_MFMA_CASES = [
    dict(fmt="NCHW4_NCHW", n=3, ic=32, ih=20, iw=20, oc=150, fh=3, pad=1),           # several tiles both ways, ragged channels
    dict(fmt="NCHW4_NCHW", n=2, ic=16, ih=23, iw=20, oc=37, fh=3, pad=1),            # oc % 4 != 0: a quad that ends early
    dict(fmt="NCHW4_NCHW", n=2, ic=64, ih=12, iw=16, oc=24, fh=1),                    # pointwise fast path
    dict(fmt="NCHW4_NCHW", n=1, ic=8, ih=31, iw=9, oc=1000, fh=5, pad=2, stride=2),   # a classifier-like tail: many channels
]


@pytest.mark.parametrize("i", range(len(NCHW4_NCHW_MFMA_CASES)))
def test_nchw4_nchw_on_the_mfma_kernel(oracle, i):
    """The planar epilogue of the register-staged tiles: QuantizedS8 dst bit-exact in every requantisation form, with
    channel, full-shape and no bias; Float32 dst exact where float arithmetic is exact and to the reference checker's
    tolerance elsewhere.  The heuristic takes the MFMA algorithm for dense problems of this format."""
    c = NCHW4_NCHW_MFMA_CASES[i]
    names = lib.tile_names()
    d = mk(c, nonline="RELU", **S)
    assert ops.conv_bias_query(d)[0].id == IGEMM
    usable = [t for t in range(len(names)) if lib.tile_usable(d, t)]
    assert [names[t] for t in usable] == ["128x128x64", "64x64x128"]
    for tile in usable:
        for nl in ("IDENTITY", "RELU", "H_SWISH"):
            for has_z in (False, True):
                tag = "nchw4_nchw mfma %s" % names[tile]
                check_case(oracle, mk(c, nonline=nl, has_z=has_z, **S), seed=140 + i, algo=IGEMM, tile=tile, tag=tag)
                check_case(oracle, mk(c, nonline=nl, has_z=has_z, dst_dtype=_abi.DT_F32, scale_bias=0.0173, scale_z=0.0041),
                           seed=160 + i, algo=IGEMM, tile=tile, tag=tag + " f32")
        # scales outside the divide-free forms (the literal chain), a full-shape bias, no bias
        check_case(oracle, mk(c, nonline="H_SWISH", has_z=True, scale_bias=3.1e-7, scale_z=1e-6, scale_dst=2.9e-6), seed=170 + i,
                   algo=IGEMM, tile=tile, tag="nchw4_nchw mfma literal chain")
        check_case(oracle, mk(c, nonline="RELU", has_z=True, bias_mode=_abi.BIAS_FULL, **S), seed=171 + i, algo=IGEMM, tile=tile,
                   tag="nchw4_nchw mfma full bias")
        check_case(oracle, mk(c, nonline="IDENTITY", bias_mode=_abi.BIAS_NONE, **S), seed=172 + i, algo=IGEMM, tile=tile,
                   tag="nchw4_nchw mfma no bias")
        check_case(oracle, mk(c, nonline="RELU", has_z=True, bias_mode=_abi.BIAS_FULL, dst_dtype=_abi.DT_F32, scale_bias=0.0173,
                              scale_z=0.0041), seed=173 + i, algo=IGEMM, tile=tile, tag="nchw4_nchw mfma f32 full bias")
        # exact: unit scales, so every float product and partial sum is a small integer
        d = mk(c, nonline="RELU", has_z=True, dst_dtype=_abi.DT_F32, scale_bias=1.0, scale_z=0.5)
        src, flt, bias, z = util.make_tensors(d, seed=180 + i, src_range=(-8, 8), flt_range=(-8, 8))
        want = oracle.conv_bias(d, src, flt, bias, z)
        got = run_gpu(d, src, flt, bias, z, algo=IGEMM, tile=tile)
        assert np.array_equal(got, want)
    # what stays on the generic kernel: a QuantizedS32 destination, groups whose filter pieces are not 16-byte aligned
    assert ops.conv_bias_query(mk(NCHW4_NCHW_CASES[3], **S))[0].id == DIRECT
    assert ops.conv_bias_query(mk(c, dst_dtype=_abi.DT_QS32, scale_bias=2e-4, scale_dst=2e-4))[0].id == DIRECT


NCHW4_NCHW_GROUP_CASES = [
    dict(fmt="NCHW4_NCHW", n=2, ic=32, ih=12, iw=12, oc=24, fh=3, group=2, pad=1),     # ocpg = 12
    dict(fmt="NCHW4_NCHW", n=3, ic=64, ih=9, iw=11, oc=40, fh=3, group=4, pad=1),      # icpg = 16, ocpg = 10: ragged quads
    dict(fmt="NCHW4_NCHW", n=2, ic=48, ih=8, iw=8, oc=96, fh=1, group=3),               # pointwise groups
]


@pytest.mark.parametrize("i", range(len(NCHW4_NCHW_GROUP_CASES)))
def test_nchw4_nchw_groups_one_dense_launch_per_group(oracle, i):
    c = NCHW4_NCHW_GROUP_CASES[i]
    assert ops.conv_bias_query(mk(c, nonline="RELU", **S))[0].id == IGEMM
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            check_case(oracle, mk(c, nonline=nl, has_z=has_z, **S), seed=240 + i, algo=IGEMM, tag="nchw4_nchw group")
            check_case(oracle, mk(c, nonline=nl, has_z=has_z, dst_dtype=_abi.DT_F32, scale_bias=0.0173, scale_z=0.0041),
                       seed=250 + i, algo=IGEMM, tag="nchw4_nchw group f32")
    check_case(oracle, mk(c, nonline="RELU", bias_mode=_abi.BIAS_NONE, **S), seed=260 + i, algo=IGEMM, tag="nchw4_nchw group no bias")
    # a full-shape bias with groups stays on the generic kernel
    assert ops.conv_bias_query(mk(c, bias_mode=_abi.BIAS_FULL, **S))[0].id == DIRECT


def test_direct_s32_dst_and_full_bias(oracle, kats):
    # the reference KAT itself, on the GPU (QuantizedS32 dst and z)
    k = kats["conv_bias_quantized8x8x32"]
    d = _abi.make_conv_desc("NCHW", 1, 1, 4, 4, 3, 3, has_z=True, dst_dtype=_abi.DT_QS32,
                            scale_bias=float(np.float32(0.02)), scale_z=float(np.float32(0.3)),
                            scale_dst=float(np.float32(0.1) * np.float32(0.2)))
    say("case KAT conv_bias_quantized8x8x32 on GPU")
    got = run_gpu(d, np.array(k["src"], np.int8).reshape(1, 1, 4, 4), np.array(k["filter"], np.int8).reshape(3, 1, 3, 3),
                  np.array(k["bias"], np.int32).reshape(1, 3, 1, 1), np.array(k["z"], np.int32).reshape(1, 3, 2, 2),
                  algo=DIRECT)
    assert got.reshape(-1).tolist() == k["dst"]
    check_case(oracle, _abi.make_conv_desc("NCHW4", 2, 8, 5, 5, 8, 3, pad=1, bias_mode=_abi.BIAS_FULL, **S), algo=DIRECT)
    check_case(oracle, _abi.make_conv_desc("NCHW4", 2, 8, 5, 5, 8, 3, pad=1, bias_mode=_abi.BIAS_NONE, **S), algo=DIRECT)
    check_case(oracle, _abi.make_conv_desc("NCHW32", 1, 32, 5, 5, 32, 3, pad=1, dst_dtype=_abi.DT_QS32,
                                           scale_bias=2e-4, scale_dst=2e-4), algo=DIRECT)


def test_s32_dst_in_place_semantics(oracle):
    """QuantizedS32 dst: raw sums for IDENTITY without z (also beyond 2^24, also with a dst scale that differs from
    the bias scale), the scale of dst everywhere else."""
    src = np.array([1, 2, 3, 5], np.int8).reshape(1, 1, 2, 2)
    flt = np.ones((1, 1, 1, 1), np.int8)
    bias = np.array([3 << 24], np.int32).reshape(1, 1, 1, 1)
    for s_b, s_d in ((2e-4, 2e-4), (2e-4, 2.0000001e-4), (1.0, 0.37)):
        d = _abi.make_conv_desc("NCHW", 1, 1, 2, 2, 1, 1, dst_dtype=_abi.DT_QS32, scale_bias=s_b, scale_dst=s_d)
        say("case s32 raw", s_b, s_d)
        got = run_gpu(d, src, flt, bias, None, algo=DIRECT)
        assert got.reshape(-1).tolist() == [50331649, 50331650, 50331651, 50331653]
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for z in (False, True):
            d = _abi.make_conv_desc("NCHW32", 2, 64, 6, 6, 32, 3, pad=1, nonline=nl, has_z=z, dst_dtype=_abi.DT_QS32,
                                    scale_bias=2e-4, scale_z=3e-4, scale_dst=2.0000001e-4)
            check_case(oracle, d, seed=91, tag="s32 " + nl, bias_range=(-(1 << 26), 1 << 26), z_range=(-100000, 100000))


def test_misaligned_tensors_take_the_generic_kernel(oracle):
    """Views at a 4-byte offset and a batch stride that is no multiple of 16: the heuristic's choice is replaced by the
    generic kernel (the reference accepts any pointer); an algorithm asked for by id reports an error instead."""
    d = _abi.make_conv_desc("NCHW32", 2, 64, 7, 7, 64, 3, pad=1, nonline="RELU", has_z=True, **S)
    src, flt, bias, z = util.make_tensors(d, seed=5)
    want = oracle.conv_bias(d, src, flt, bias, z)

    def shifted(x, extra=0):
        flat = torch.zeros(x.size + 64 + extra, dtype=torch.int8, device="cuda")
        flat[4:4 + x.size] = torch.from_numpy(x.reshape(-1)).cuda()
        return flat, flat[4:4 + x.size].view(*x.shape)

    algo, _ = ops.conv_bias_query(d)
    assert algo.id == IGEMM
    for which in ("src", "z", "dst"):
        say("case misaligned", which)
        t = dict(src=to_dev(src), z=to_dev(z), dst=torch.empty(want.shape, dtype=torch.int8, device="cuda"))
        keep, t[which] = shifted(dict(src=src, z=z, dst=want)[which])
        assert t[which].data_ptr() % 16 == 4
        rc = lib.lib().mi355_convbias_s8_exec(ops._stream(), d, algo, ops._ptr(t["src"]), ops._ptr(to_dev(flt)),
                                             ops._ptr(to_dev(bias)), ops._ptr(t["z"]), ops._ptr(t["dst"]), None, 0)
        assert rc == 0, lib.lib().mi355_last_error()
        torch.cuda.synchronize()
        assert np.array_equal(t["dst"].cpu().numpy(), want)
        forced, _ = ops.conv_bias_query(d, IGEMM)
        rc = lib.lib().mi355_convbias_s8_exec(ops._stream(), d, forced, ops._ptr(t["src"]), ops._ptr(to_dev(flt)),
                                             ops._ptr(to_dev(bias)), ops._ptr(t["z"]), ops._ptr(t["dst"]), None, 0)
        assert rc == _abi.ERR_ALGO
    # a batch stride that is not a multiple of 16 bytes
    per = src[0].size
    d2 = _abi.make_conv_desc("NCHW32", 2, 64, 7, 7, 64, 3, pad=1, nonline="RELU", has_z=True, src_stride_n=per + 4, **S)
    check_case(oracle, d2, seed=5, tag="odd batch stride")


def test_direct_exact_epilogue_for_odd_scales(oracle):
    """Scales outside the fast form's envelope take the literal IEEE-divide epilogue."""
    for sd in (1e-20, 3e15):
        d = _abi.make_conv_desc("NCHW4", 1, 8, 5, 5, 8, 3, pad=1, nonline="H_SWISH", has_z=True, scale_bias=2e-4,
                                scale_z=0.05, scale_dst=sd)
        check_case(oracle, d, algo=None, tag="oddscale")


# ---------------------------------------------------------------------------------------------
# MFMA implicit GEMM
# ---------------------------------------------------------------------------------------------

IGEMM_CASES = [
    # fmt, n, ic, ih, iw, oc, f, pad, stride
    ("NCHW32", 2, 64, 8, 8, 64, 1, 0, 1),
    ("NCHW32", 3, 32, 7, 7, 96, 1, 0, 1),       # ragged pixels (147) and oc = 96
    ("NCHW32", 2, 64, 9, 11, 64, 3, 1, 1),
    ("NCHW32", 2, 96, 12, 12, 160, 3, 1, 2),
    ("NCHW32", 1, 32, 14, 14, 32, 5, 2, 1),
    ("NCHW32", 1, 32, 17, 15, 64, 7, 3, 2),
    ("NCHW32", 2, 128, 6, 6, 256, 1, 0, 2),     # strided 1x1 (downsample)
    ("NCHW32", 1, 256, 5, 5, 320, 3, 0, 1),     # no padding, long K
    ("NCHW4", 2, 16, 9, 9, 32, 1, 0, 1),
    ("NCHW4", 2, 64, 10, 10, 64, 3, 1, 1),      # cfg0 family
    ("NCHW4", 1, 4, 30, 30, 64, 7, 3, 2),       # stem: K = 196 bytes, not a multiple of 32
    ("NCHW4", 2, 24, 8, 8, 144, 1, 0, 1),       # MobileNetV2 expand
    ("NCHW4", 2, 144, 8, 8, 24, 1, 0, 1),       # MobileNetV2 project (oc < 32)
    ("NCHW4", 1, 12, 9, 7, 20, 3, 1, 2),        # oc % 32 != 0, K = 108
    ("NCHW4", 3, 40, 7, 7, 40, 1, 0, 1),        # 4-packed pointwise: K = 40 and oc = 40 ragged, 147 pixels, images of 49
    ("NCHW4", 2, 96, 9, 9, 24, 1, 0, 2),        # 4-packed pointwise, stride 2, narrow output
    ("NCHW4", 2, 192, 6, 6, 72, 1, 0, 1),       # 4-packed pointwise, several k-stages
    ("NCHW4", 2, 64, 9, 9, 96, 1, 0, 2),        # 4-packed pointwise, 64 channels in (two k-steps), stride 2
    ("NCHW4", 2, 100, 7, 7, 128, 1, 0, 1),      # streaming kernel: four k-steps, the last one ragged
    ("NCHW4", 1, 160, 7, 7, 640, 1, 0, 1),      # streaming kernel: five k-steps, 20 channel blocks
    ("NCHW4_NCHW32", 2, 16, 8, 8, 64, 3, 1, 1),
    ("NCHW32_NCHW4", 2, 64, 8, 8, 24, 3, 1, 1),
]


@pytest.mark.parametrize("i", range(len(IGEMM_CASES)))
def test_igemm_formats_and_tiles(oracle, i):
    fmt, n, ic, ih, iw, oc, f, pad, stride = IGEMM_CASES[i]
    mixed = "_" in fmt
    from megengine_amd import lib
    ntiles = len(lib.tile_names())
    for tile in range(ntiles):
        nl = ("IDENTITY", "RELU", "H_SWISH")[(tile + i) % 3]
        has_z = (not mixed) and (tile % 2 == 0)
        d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, pad=pad, stride=stride, nonline=nl, has_z=has_z, **S)
        check_case(oracle, d, seed=100 + i, algo=IGEMM, tile=tile, tag="igemm%d" % i)


def test_igemm_long_k_table(oracle):
    """3x3 over 1024 channels of a 4-packed tensor: 2304 k-units, beyond the first 2048 table entries."""
    d = _abi.make_conv_desc("NCHW4", 1, 1024, 6, 6, 64, 3, pad=1, nonline="RELU", **S)
    a, _ = ops.conv_bias_query(d)
    assert a.id == IGEMM
    check_case(oracle, d, seed=77, algo=IGEMM, tag="longk4")
    d = _abi.make_conv_desc("NCHW32", 1, 8192, 3, 3, 32, 3, pad=1, nonline="IDENTITY", **S)
    check_case(oracle, d, seed=78, algo=IGEMM, tag="longk32")


def test_igemm_nonlines_z_bias(oracle):
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            for bm in (_abi.BIAS_BROADCAST_CHANNEL, _abi.BIAS_NONE):
                d = _abi.make_conv_desc("NCHW32", 2, 64, 10, 10, 64, 3, pad=1, nonline=nl, has_z=has_z, bias_mode=bm, **S)
                check_case(oracle, d, seed=7, algo=IGEMM, tag="nlzb")
                d = _abi.make_conv_desc("NCHW4", 2, 32, 10, 10, 40, 3, pad=1, nonline=nl, has_z=has_z, bias_mode=bm, **S)
                check_case(oracle, d, seed=8, algo=IGEMM, tag="nlzb4")


def test_igemm_saturation_and_scales(oracle):
    """Big accumulators (full-range int8 x long K) saturate both ways; random per-tensor scales."""
    rng = np.random.RandomState(3)
    for t in range(6):
        sb = float(np.float32(np.exp(rng.uniform(np.log(1e-6), np.log(2.5e-3)))))
        sz = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        sd = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        d = _abi.make_conv_desc("NCHW32", 1, 256, 6, 6, 64, 3, pad=1, nonline=("IDENTITY", "RELU", "H_SWISH")[t % 3],
                                has_z=True, scale_bias=sb, scale_z=sz, scale_dst=sd)
        check_case(oracle, d, seed=40 + t, algo=IGEMM, tag="scales")


def test_igemm_strided_batch(oracle):
    d0 = _abi.make_conv_desc("NCHW32", 3, 64, 6, 6, 64, 3, pad=1, nonline="RELU", has_z=True, **S)
    per_src, per_dst = 64 * 36, 64 * 36
    d = _abi.make_conv_desc("NCHW32", 3, 64, 6, 6, 64, 3, pad=1, nonline="RELU", has_z=True,
                            src_stride_n=per_src + 64, z_stride_n=per_dst + 32, dst_stride_n=per_dst + 96, **S)
    want = check_case(oracle, d, seed=5, algo=IGEMM, tag="strided")
    assert np.array_equal(want, check_case(oracle, d0, seed=5, algo=IGEMM, tag="dense"))


def test_config0_full_size(oracle):
    """Workload config 0: NCHW4 N16 64->64 56x56 3x3 s1 p1, bias U[-1000,1000], RELU, scales .02*.01 -> .05."""
    sb = float(np.float32(0.02) * np.float32(0.01))
    d = _abi.make_conv_desc("NCHW4", 16, 64, 56, 56, 64, 3, pad=1, nonline="RELU", scale_bias=sb,
                            scale_dst=float(np.float32(0.05)))
    check_case(oracle, d, seed=2024, tag="config0")


# ---------------------------------------------------------------------------------------------
# depthwise
# ---------------------------------------------------------------------------------------------

DW_CASES = [
    # fmt, n, c, ih, iw, f, pad, stride
    ("NCHW4", 2, 32, 14, 14, 3, 1, 1),
    ("NCHW4", 2, 24, 15, 13, 3, 1, 2),
    ("NCHW4", 1, 96, 28, 28, 3, 1, 1),
    ("NCHW4", 1, 96, 28, 28, 3, 1, 2),
    ("NCHW44", 2, 16, 7, 7, 3, 1, 1),      # ow % 4 != 0
    ("NCHW4", 1, 8, 12, 12, 5, 2, 1),      # generic filter size
    ("NCHW4", 1, 8, 9, 16, 3, 0, 1),       # no padding
    ("NCHW44", 1, 8, 11, 11, 3, 1, 3),     # generic stride
    ("NCHW4", 1, 8, 15, 9, 3, 1, 1),       # odd output height: the last row strip is half empty
    ("NCHW4", 1, 8, 10, 10, 3, 0, 2),      # stride 2 without padding
    ("NCHW4", 1, 8, 9, 9, 3, 2, 1),        # padding wider than the filter radius
    ("NCHW4", 3, 12, 5, 5, 3, 1, 2),       # planes much smaller than a wavefront
    ("NCHW4", 2, 8, 6, 37, 3, 1, 1),       # ragged row ends (iw % 4 = 1)
]


@pytest.mark.parametrize("i", range(len(DW_CASES)))
def test_depthwise(oracle, i):
    fmt, n, c, ih, iw, f, pad, stride = DW_CASES[i]
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            d = _abi.make_conv_desc(fmt, n, c, ih, iw, c, f, group=c, pad=pad, stride=stride, nonline=nl, has_z=has_z, **S)
            a, _ = ops.conv_bias_query(d)
            assert a.id == DW
            check_case(oracle, d, seed=200 + i, tag="dw%d" % i)
    # scales outside the range of the divide-free epilogue: the kernel must take the literal chain
    d = _abi.make_conv_desc(fmt, n, c, ih, iw, c, f, group=c, pad=pad, stride=stride, nonline="RELU", has_z=True,
                            scale_bias=1e-20, scale_z=3e-19, scale_dst=1e-18)
    check_case(oracle, d, seed=300 + i, tag="dw%d-literal" % i)


# ---------------------------------------------------------------------------------------------
# chooser + cross-algorithm agreement at larger sizes
# ---------------------------------------------------------------------------------------------

def test_heuristic_picks(oracle):
    d = _abi.make_conv_desc("NCHW32", 64, 256, 56, 56, 64, 1)
    assert ops.conv_bias_query(d)[0].id == IGEMM
    d = _abi.make_conv_desc("NCHW", 1, 8, 8, 8, 8, 3, pad=1)
    assert ops.conv_bias_query(d)[0].id == DIRECT
    d = _abi.make_conv_desc("NCHW4", 1, 32, 8, 8, 32, 3, pad=1, group=32)
    assert ops.conv_bias_query(d)[0].id == DW
    # group convolution over whole 32-channel blocks runs on the MFMA kernel (second-generation tiles); groups that
    # split a channel block stay on the generic kernel
    d = _abi.make_conv_desc("NCHW32", 1, 64, 8, 8, 64, 3, pad=1, group=2)
    a = ops.conv_bias_query(d)[0]
    assert a.id == IGEMM and lib.tile_names()[a.tile_cfg].startswith("v2_")
    # NCHW4 groups of whole blocks of 4: the dense MFMA tiles, one launch per group; groups that split a block of 4 do
    # not exist in the format (dnn/src/common/convolution.cpp:392-407)
    d = _abi.make_conv_desc("NCHW4", 1, 32, 8, 8, 32, 3, pad=1, group=4)
    assert ops.conv_bias_query(d)[0].id == IGEMM
    # plain NCHW: relayout + MFMA through the workspace once the problem pays for the extra launches
    d = _abi.make_conv_desc("NCHW", 8, 64, 28, 28, 64, 3, pad=1)
    a, ws = ops.conv_bias_query(d)
    assert lib.algo_names()[a.id] == "MI355_NCHW_RELAYOUT_MFMA_I8" and ws > 0
    # 4-packed pointwise layers at batch 64: streaming kernel for the expansions and the narrow projections, LDS-direct
    # tiles for the long reductions on few pixels, register-staged tiles elsewhere
    names = lib.tile_names()
    for (ic, hw, oc), want in (((16, 112, 96), "pw4_stream"), ((96, 56, 24), "pw4_stream"), ((384, 14, 64), "dma4_64x64x128"),
                               ((160, 7, 960), "dma4_128x64x128"), ((96, 14, 576), "128x128x64")):
        a, _ = ops.conv_bias_query(_abi.make_conv_desc("NCHW4", 64, ic, hw, hw, oc, 1))
        assert a.id == IGEMM and names[a.tile_cfg] == want, (ic, hw, oc, names[a.tile_cfg])
    # 32-packed layers of ResNet-50 at batch 64 for a caller that pre-processes the filter: second-generation tiles, and
    # the patch-staged tile for the 3x3 layers over 256 channels
    S8 = dict(scale_bias=2e-4, scale_z=0.05, scale_dst=0.05, nonline="RELU")
    for (ic, hw, oc, f), want in (((256, 14, 256, 3), "v3_128x128x256r3"), ((1024, 14, 256, 1), "v2_64x128x128r3"),
                                  ((64, 56, 64, 3), "v2_64x128x64r4"), ((512, 7, 512, 3), "v2_64x64x128r4")):
        a, _ = ops.conv_bias_query(_abi.make_conv_desc("NCHW32", 64, ic, hw, hw, oc, f, pad=f // 2, **S8),
                                   _abi.ALGO_HEURISTIC_PREPROCESS)
        assert a.id == IGEMM and names[a.tile_cfg] == want, (ic, hw, oc, f, names[a.tile_cfg])
    # pointwise over 64 channels on both sides: the streaming kernel, with or without weight pre-processing
    for req in (_abi.ALGO_HEURISTIC, _abi.ALGO_HEURISTIC_PREPROCESS):
        a, _ = ops.conv_bias_query(_abi.make_conv_desc("NCHW32", 64, 64, 56, 56, 64, 1, **S8), req)
        assert a.id == IGEMM and names[a.tile_cfg] == "pw32_stream", names[a.tile_cfg]
    # the same 3x3 over 64 channels at batch 128, five tiles per workgroup: the weight-resident tile
    a, _ = ops.conv_bias_query(_abi.make_conv_desc("NCHW32", 128, 64, 56, 56, 64, 3, pad=1, **S8), _abi.ALGO_HEURISTIC_PREPROCESS)
    assert a.id == IGEMM and names[a.tile_cfg] == "v4_64x128res", names[a.tile_cfg]


def test_general_epilogue_on_the_mfma_kernel(oracle):
    """QuantizedS32 dst (the reference's default dst dtype for s8 x s8, dnn/src/common/convolution.cpp:555-574), full-shape
    bias and scales outside the fast forms' envelope run the MFMA kernel (second-generation tiles) on 32-packed inputs."""
    names = lib.tile_names()
    v2 = [i for i, n in enumerate(names) if n.startswith("v2_")]
    cases = [
        dict(dst_dtype=_abi.DT_QS32, scale_bias=2e-4, scale_dst=2e-4),
        dict(dst_dtype=_abi.DT_QS32, nonline="RELU", scale_bias=2e-4, scale_dst=2.0000001e-4),
        dict(dst_dtype=_abi.DT_QS32, nonline="H_SWISH", scale_bias=2e-4, scale_dst=2e-4),
        dict(bias_mode=_abi.BIAS_FULL, nonline="RELU", has_z=True, **S),
        dict(bias_mode=_abi.BIAS_FULL, nonline="IDENTITY", scale_bias=1.3e-3, scale_dst=0.0271),
        dict(nonline="H_SWISH", has_z=True, scale_bias=2e-4, scale_z=0.05, scale_dst=1e-20),
        dict(nonline="RELU", scale_bias=2e-4, scale_dst=3e15),
        # a QuantizedS32 residual on a QuantizedS32 dst (z has the dtype of dst, dnn/src/common/conv_bias.cpp:127-132)
        dict(dst_dtype=_abi.DT_QS32, has_z=True, scale_bias=2e-4, scale_z=3e-4, scale_dst=2e-4),
        dict(dst_dtype=_abi.DT_QS32, has_z=True, nonline="RELU", scale_bias=2e-4, scale_z=1e-4, scale_dst=2e-4),
    ]
    shapes = [("NCHW32", 2, 64, 9, 11, 96, 3, 1, 1, 1), ("NCHW32", 3, 128, 7, 7, 64, 1, 0, 1, 1), ("NCHW32", 2, 128, 8, 8, 128, 3, 1, 2, 2),
              ("NCHW32_NCHW4", 2, 64, 8, 8, 24, 3, 1, 1, 1)]
    for ci, kw in enumerate(cases):
        for si, (fmt, n, ic, ih, iw, oc, f, pad, stride, group) in enumerate(shapes):
            if fmt == "NCHW32_NCHW4" and kw.get("has_z"):
                continue
            d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, pad=pad, stride=stride, group=group, **kw)
            a, _ = ops.conv_bias_query(d)
            assert a.id == IGEMM and names[a.tile_cfg].startswith("v2_"), (ci, si, names[a.tile_cfg])
            big = dict(bias_range=(-(1 << 26), 1 << 26), z_range=(-(1 << 24), 1 << 24)) if kw.get("dst_dtype") == _abi.DT_QS32 else {}
            check_case(oracle, d, seed=900 + 10 * ci + si, tag="general %d/%d heuristic" % (ci, si), **big)
            for tile in v2[::3]:
                check_case(oracle, d, seed=900 + 10 * ci + si, algo=IGEMM, tile=tile, tag="general %d/%d %s" % (ci, si, names[tile]), **big)
    # 4-packed inputs with a QuantizedS32 dst stay on the generic kernel
    d = _abi.make_conv_desc("NCHW4", 1, 64, 6, 6, 64, 3, pad=1, dst_dtype=_abi.DT_QS32, scale_bias=2e-4, scale_dst=2e-4)
    assert ops.conv_bias_query(d)[0].id == DIRECT


def test_preprocessed_filter_equals_plain_filter(oracle):
    """exec with a PreprocessedFilter == exec with the filter, bit for bit, for every tile that has a pre-processed form;
    tiles without one report size 0 (nothing to hoist) and refuse exec_preprocessed."""
    names = lib.tile_names()
    n_pre = 0
    for ci, (fmt, n, ic, ih, iw, oc, f, pad, stride) in enumerate(IGEMM_CASES):
        for nl, z in (("RELU", True), ("IDENTITY", False)):
            if z and fmt in ("NCHW4_NCHW32", "NCHW32_NCHW4"):
                continue
            d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, pad=pad, stride=stride, nonline=nl, has_z=z, **S)
            src, flt, bias, zz = util.make_tensors(d, seed=700 + ci)
            dev = [to_dev(x) for x in (src, flt, bias, zz)]
            for tile in range(len(names)):
                if not lib.tile_usable(d, tile):
                    continue
                a, _ = ops.conv_bias_query(d, IGEMM)
                a.tile_cfg = tile
                pre = ops.conv_bias_preprocess(d, dev[1], a)
                if pre is None:
                    assert not (names[tile].startswith(("v2_", "v3_")) and fmt in ("NCHW32", "NCHW32_NCHW4"))
                    continue
                assert names[tile].startswith(("v2_", "v3_"))  # the patch-staged tiles read the same filter form
                say("case preprocessed", fmt, n, ic, ih, iw, oc, f, pad, stride, nl, z, names[tile])
                plain = ops.conv_bias_exec(d, dev[0], dev[1], dev[2], dev[3], algo=a)
                got = ops.conv_bias_exec_preprocessed(d, dev[0], pre, dev[2], dev[3], algo=a)
                torch.cuda.synchronize()
                assert torch.equal(got, plain), names[tile]
                n_pre += 1
    assert n_pre > 0
    # group convolution with a pre-processed filter, against the checker
    d = _abi.make_conv_desc("NCHW32", 2, 128, 9, 9, 192, 3, pad=1, group=2, nonline="H_SWISH", has_z=True, **S)
    src, flt, bias, zz = util.make_tensors(d, seed=777)
    want = oracle.conv_bias(d, src, flt, bias, zz)
    a, _ = ops.conv_bias_query(d)
    pre = ops.conv_bias_preprocess(d, to_dev(flt), a)
    assert pre is not None
    got = ops.conv_bias_exec_preprocessed(d, to_dev(src), pre, to_dev(bias), to_dev(zz), algo=a)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    # an algorithm without a pre-processed form
    a, _ = ops.conv_bias_query(d, DIRECT)
    assert ops.conv_bias_preprocess(d, to_dev(flt), a) is None


NCHW_MFMA_CASES = [
    # the generic kernel's NCHW shapes (DIRECT_CASES) scaled up until the relayout + MFMA algorithm is the heuristic's
    # choice; channel counts that are no multiple of 32 (zero-padded blocks on either side), ragged images
    dict(n=4, ic=24, ih=28, iw=28, oc=40, fh=3, pad=1),
    dict(n=16, ic=3, ih=57, iw=49, oc=5, fh=3, pad=1),                     # DIRECT_CASES[0] at 8x the image and the batch
    dict(n=3, ic=64, ih=14, iw=14, oc=128, fh=1),                           # whole blocks, 196 pixels (no vector path)
    dict(n=2, ic=32, ih=32, iw=32, oc=64, fh=3, pad=1, stride=2),           # every relayout on its vector path
    dict(n=2, ic=20, ih=19, iw=23, oc=36, fh=5, fw=3, pad=(2, 1), stride=(2, 1)),
    dict(n=2, ic=64, ih=16, iw=16, oc=128, fh=3, pad=1, group=2),           # groups of whole 32-channel blocks
    dict(n=1, ic=100, ih=30, iw=30, oc=7, fh=3),
]


@pytest.mark.parametrize("i", range(len(NCHW_MFMA_CASES)))
def test_plain_nchw_on_the_mfma_kernel(oracle, i):
    """Format::NCHW through relayout -> NCHW32 MFMA kernel -> relayout in the caller's workspace, against the checker's
    NCHW path, every activation, with and without a residual; the generic kernel must give the same tensor."""
    c = NCHW_MFMA_CASES[i]
    nchw = lib.algo_names().index("MI355_NCHW_RELAYOUT_MFMA_I8")
    for nl, has_z in (("RELU", True), ("IDENTITY", False), ("H_SWISH", True)):
        d = mk(dict(c, fmt="NCHW"), nonline=nl, has_z=has_z, **S)
        a, ws = ops.conv_bias_query(d)
        assert a.id == nchw and ws > 0, (i, a.id, ws)
        want = check_case(oracle, d, seed=1200 + i, algo=nchw, tag="nchw-mfma %d" % i)
        check_case(oracle, d, seed=1200 + i, algo=DIRECT, tag="nchw-direct %d" % i)
        assert want is not None


def test_plain_nchw_workspace_contract(oracle):
    """check_exec's workspace rule (dnn/src/common/conv_bias.cpp:32-37): exec with less than query reported is
    MI355_ERR_WORKSPACE and launches nothing; a caller without a workspace gets the generic kernel from the heuristic;
    exactly the reported size is enough, and a larger, offset workspace works as well."""
    nchw = lib.algo_names().index("MI355_NCHW_RELAYOUT_MFMA_I8")
    d = _abi.make_conv_desc("NCHW", 4, 24, 28, 28, 40, 3, pad=1, nonline="RELU", has_z=True, **S)
    src, flt, bias, z = util.make_tensors(d, seed=77)
    want = oracle.conv_bias(d, src, flt, bias, z)
    dev = [to_dev(x) for x in (src, flt, bias, z)]
    a, ws = ops.conv_bias_query(d)
    assert a.id == nchw
    L = lib.lib()
    dst = torch.full(want.shape, 99, dtype=torch.int8, device="cuda")
    short = torch.empty(ws - 256, dtype=torch.uint8, device="cuda")
    rc = L.mi355_convbias_s8_exec(ops._stream(), d, a, *[ops._ptr(t) for t in dev], ops._ptr(dst), ops._ptr(short), short.numel())
    assert rc == _abi.ERR_WORKSPACE, L.mi355_last_error()
    rc = L.mi355_convbias_s8_exec(ops._stream(), d, a, *[ops._ptr(t) for t in dev], ops._ptr(dst), None, 0)
    assert rc == _abi.ERR_WORKSPACE
    torch.cuda.synchronize()
    assert int((dst != 99).sum()) == 0          # nothing was launched
    # no algorithm given and no workspace: the heuristic inside exec stays within what the caller brought
    rc = L.mi355_convbias_s8_exec(ops._stream(), d, None, *[ops._ptr(t) for t in dev], ops._ptr(dst), None, 0)
    assert rc == 0, L.mi355_last_error()
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), want)
    exact = torch.empty(ws, dtype=torch.uint8, device="cuda")
    got = ops.conv_bias_exec(d, *dev, algo=a, workspace=exact)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    big = torch.empty(ws + 4096, dtype=torch.uint8, device="cuda")
    got = ops.conv_bias_exec(d, *dev, algo=a, workspace=big[1024:])
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    # tensors that are not 16-byte aligned: the relayouts take any pointer
    flat = torch.zeros(src.size + 64, dtype=torch.int8, device="cuda")
    flat[4:4 + src.size] = dev[0].reshape(-1)
    got = ops.conv_bias_exec(d, flat[4:4 + src.size].view(*src.shape), dev[1], dev[2], dev[3], algo=a)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)


NCHW4_GROUP_CASES = [
    dict(n=1, ic=60, ih=9, iw=9, oc=20, fh=3, group=5, pad=1),      # shape family of dnn/test/naive/convolution.cpp:141-220
    dict(n=20, ic=60, ih=30, iw=30, oc=20, fh=3, group=5),          # ... at the reference's own size {20,15,30,30,4} x {5,4,3,3,3,4}
    dict(n=2, ic=32, ih=14, iw=14, oc=64, fh=3, group=4, pad=1, stride=2),
    dict(n=3, ic=48, ih=10, iw=12, oc=24, fh=1, group=2),
    dict(n=2, ic=256, ih=8, iw=8, oc=256, fh=3, group=8, pad=1),
]


@pytest.mark.parametrize("i", range(len(NCHW4_GROUP_CASES)))
def test_nchw4_group_convolution_one_dense_launch_per_group(oracle, i):
    c = NCHW4_GROUP_CASES[i]
    for nl, has_z in (("RELU", True), ("IDENTITY", False), ("H_SWISH", True)):
        d = mk(dict(c, fmt="NCHW4"), nonline=nl, has_z=has_z, **S)
        assert ops.conv_bias_query(d)[0].id == IGEMM
        check_case(oracle, d, seed=1300 + i, tag="nchw4 group %d heuristic" % i)
        names = lib.tile_names()
        for tile in range(0, len(names), 5):
            check_case(oracle, d, seed=1300 + i, algo=IGEMM, tile=tile, tag="nchw4 group %d %s" % (i, names[tile]))
    # batch-strided views of a group convolution: the per-group views keep the strides of the whole tensors
    ss, fs, bs, ds = _abi.conv_shapes(mk(dict(c, fmt="NCHW4")))
    kw = dict(src_stride_n=int(np.prod(ss[1:])) + 32, dst_stride_n=int(np.prod(ds[1:])) + 16, z_stride_n=int(np.prod(ds[1:])) + 48)
    d = mk(dict(c, fmt="NCHW4"), nonline="RELU", has_z=True, **S, **kw)
    check_case(oracle, d, seed=1350 + i, tag="nchw4 group %d strided batch" % i)


def test_forced_tile_that_cannot_run_is_an_error(oracle):
    """exec runs the tile it is given or refuses: a tile the caller named and that is no algorithm for the problem is
    MI355_ERR_ALGO (so a fast-run chooser never times one kernel under two names); the same tile under the heuristic's
    flag is replaced by the one that can run."""
    names = lib.tile_names()
    d = _abi.make_conv_desc("NCHW4", 2, 64, 9, 9, 64, 3, pad=1, nonline="RELU", **S)
    src, flt, bias, z = util.make_tensors(d, seed=31)
    want = oracle.conv_bias(d, src, flt, bias, z)
    dev = [to_dev(x) for x in (src, flt, bias, z)]
    bad = names.index("v2_128x128x64r4")
    assert not lib.tile_usable(d, bad)
    forced, _ = ops.conv_bias_query(d, IGEMM)
    forced.tile_cfg = bad
    with pytest.raises(lib.Mi355Error) as e:
        ops.conv_bias_exec(d, *dev, algo=forced)
    assert e.value.status == _abi.ERR_ALGO
    heur, _ = ops.conv_bias_query(d)
    assert heur.id == IGEMM
    heur.tile_cfg = bad
    got = ops.conv_bias_exec(d, *dev, algo=heur)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)


# ---------------------------------------------------------------------------------------------
# every tile configuration (register-staged and LDS-direct, 4- and 8-wave) on ragged shapes
# ---------------------------------------------------------------------------------------------

RAGGED = [
    # fmt, n, ic, ih, iw, oc, f, stride, pad, nonline, z, extra
    ("NCHW32", 3, 96, 9, 11, 96, 3, 1, 1, "RELU", True, {}),             # pixels % 32 != 0, oc % 64 != 0, K = 864
    ("NCHW32", 2, 160, 7, 7, 32, 1, 1, 0, "IDENTITY", False, {}),        # pointwise, K = 160: not a multiple of a stage
    ("NCHW32", 2, 256, 10, 10, 160, 1, 2, 0, "H_SWISH", True, {}),       # strided pointwise fast path
    ("NCHW32", 1, 64, 13, 5, 224, 5, 2, 2, "RELU", False, {}),           # 5x5 stride 2, one image
    ("NCHW32_NCHW4", 2, 64, 8, 8, 40, 3, 1, 1, "RELU", False, {}),       # 32-packed in, 4-packed out, oc % 32 != 0
    ("NCHW32", 4, 128, 6, 6, 64, 3, 1, 0, "RELU", True, {"batch_pad": 64}),  # batch-strided src / dst / z views
    ("NCHW4", 2, 24, 9, 9, 48, 3, 1, 1, "RELU", True, {}),               # 4-packed 3x3: LDS-direct ids fall back
    ("NCHW4", 3, 64, 6, 6, 64, 1, 1, 0, "RELU", True, {"batch_pad": 64}),  # 4-packed pointwise, batch-strided views
    ("NCHW4", 2, 160, 7, 7, 100, 1, 1, 0, "H_SWISH", True, {}),          # 4-packed pointwise, ragged everything
    ("NCHW4", 3, 32, 6, 6, 200, 1, 1, 0, "RELU", True, {"batch_pad": 64}),  # few channels in, 7 channel blocks out, strided views
    ("NCHW4", 5, 20, 7, 9, 36, 1, 1, 0, "IDENTITY", False, {}),          # few channels in: K = 20, oc = 36, 315 pixels
    ("NCHW4", 3, 192, 6, 6, 32, 1, 1, 0, "RELU", True, {"batch_pad": 64}),  # narrow projection with residual, six k-steps, strided views
    ("NCHW4", 2, 72, 7, 7, 20, 1, 1, 0, "H_SWISH", True, {}),            # narrow projection with residual, K = 72, oc = 20
]


@pytest.mark.parametrize("i", range(len(RAGGED)))
def test_every_tile_on_ragged_shapes(oracle, i):
    fmt, n, ic, ih, iw, oc, f, stride, pad, nl, z, extra = RAGGED[i]
    kw = dict(S)
    d0 = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, stride=stride, pad=pad, nonline=nl, has_z=z, **kw)
    if extra.get("batch_pad"):
        ss, fs, bs, ds = _abi.conv_shapes(d0)
        per_src = int(np.prod(ss[1:])) + extra["batch_pad"]
        per_dst = int(np.prod(ds[1:])) + extra["batch_pad"]
        kw.update(src_stride_n=per_src, dst_stride_n=per_dst, z_stride_n=per_dst)
    d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, stride=stride, pad=pad, nonline=nl, has_z=z, **kw)
    from megengine_amd import lib
    for tile in range(len(lib.tile_names())):
        check_case(oracle, d, seed=400 + i, algo=IGEMM, tile=tile, tag="ragged%d/%s" % (i, lib.tile_names()[tile]))


# ---------------------------------------------------------------------------------------------
# patch-staged tiles (32-packed, stride 1, filters larger than 1x1): the activations of a tile staged once per channel
# block as a patch of padded input rows
# ---------------------------------------------------------------------------------------------

PATCH_CASES = [
    # n, ic, ih, iw, oc, fh, fw, pad
    (2, 64, 14, 14, 64, 3, 3, 1),          # a tile spans both images (196 pixels each)
    (3, 32, 7, 7, 96, 3, 3, 1),            # one channel block: nothing to prefetch
    (2, 96, 9, 11, 160, 3, 3, 1),          # odd width, three channel blocks, ragged channel tile
    (1, 64, 20, 17, 64, 5, 5, 2),          # 5x5
    (2, 32, 12, 12, 32, 3, 3, 0),          # no padding
    (5, 64, 7, 7, 256, 3, 3, 1),           # five small images per tile
    (2, 64, 16, 16, 128, 3, 5, (1, 2)),    # non-square filter
    (1, 128, 30, 30, 96, 3, 3, (2, 1)),    # padding wider than the filter radius: output larger than input
    (2, 64, 56, 56, 64, 3, 3, 1),          # rows longer than a wave's pixels
    (4, 256, 14, 14, 256, 3, 3, 1),        # eight channel blocks: the patch slots recycle
    (9, 32, 5, 5, 64, 3, 3, 1),            # tiny images, ragged last tile
    (1, 32, 40, 33, 288, 5, 5, 2),         # 5x5, three channel tiles
]


@pytest.mark.parametrize("i", range(len(PATCH_CASES)))
def test_patch_staged_tiles(oracle, i):
    n, ic, ih, iw, oc, fh, fw, pad = PATCH_CASES[i]
    names = lib.tile_names()
    ran = 0
    for nl, z in (("RELU", True), ("IDENTITY", False), ("H_SWISH", True)):
        # a destination scale that keeps most outputs inside the int8 range
        d = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, fh, fw, pad=pad, nonline=nl, has_z=z, scale_bias=2e-4,
                                scale_z=0.05, scale_dst=0.05 * (ic * fh * fw / 64) ** 0.5)
        for tile, name in enumerate(names):
            if name.startswith("v3_") and check_case(oracle, d, seed=50 + i, algo=IGEMM, tile=tile,
                                                      tag="patch%d/%s" % (i, name)) is not None:
                ran += 1
    assert ran >= 3, "no patch-staged tile took case %d" % i


# ---------------------------------------------------------------------------------------------
# first-layer kernel: NCHW4 with 4 input channels, the patch-staged MFMA path
# ---------------------------------------------------------------------------------------------

C4_CASES = [
    # n, ih, iw, oc, fh, fw, stride, pad
    (2, 30, 30, 64, 7, 7, 2, 3),      # ResNet stem family
    (1, 33, 29, 32, 7, 7, 2, 3),      # odd sizes: ragged tiles in both directions, half a channel tile
    (2, 17, 40, 96, 3, 3, 2, 1),      # 3x3 stride 2 stem, two channel tiles (oc % 64 != 0)
    (1, 20, 20, 24, 3, 3, 1, 1),      # stride 1, oc % 32 != 0
    (3, 9, 9, 16, 5, 3, 1, 2),        # non-square filter, padding wider than the filter radius
    (1, 12, 50, 128, 1, 1, 1, 0),     # pointwise
    (2, 16, 16, 40, 8, 8, 2, 0),      # largest supported filter, no padding
]


@pytest.mark.parametrize("i", range(len(C4_CASES)))
def test_first_layer_kernel(oracle, i):
    n, ih, iw, oc, fh, fw, stride, pad = C4_CASES[i]
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            d = _abi.make_conv_desc("NCHW4", n, 4, ih, iw, oc, fh, fw, stride=stride, pad=pad, nonline=nl, has_z=has_z, **S)
            a, _ = ops.conv_bias_query(d)
            assert a.id == C4
            check_case(oracle, d, seed=500 + i, tag="c4-%d" % i)
    # no bias, batch-strided views
    d0 = _abi.make_conv_desc("NCHW4", n, 4, ih, iw, oc, fh, fw, stride=stride, pad=pad, nonline="RELU", has_z=True, **S)
    ss, fs, bs, ds = _abi.conv_shapes(d0)
    d = _abi.make_conv_desc("NCHW4", n, 4, ih, iw, oc, fh, fw, stride=stride, pad=pad, nonline="RELU", has_z=True,
                            bias_mode=_abi.BIAS_NONE, src_stride_n=int(np.prod(ss[1:])) + 20,
                            dst_stride_n=int(np.prod(ds[1:])) + 12, z_stride_n=int(np.prod(ds[1:])) + 36, **S)
    check_case(oracle, d, seed=600 + i, tag="c4-%d-strided" % i)


RESIDENT_CASES = [
    # n, ic, ih, iw, oc: 3x3 / stride 1 / pad 1 over 32 or 64 channels, the shapes the weight-resident tile takes
    (2, 64, 56, 56, 64),      # the ResNet-50 case: 24.5 tiles per image, the last one half full
    (3, 32, 17, 23, 96),      # odd sizes, two channel tiles (the second one half full), rows of 23 pixels
    (2, 64, 14, 14, 128),     # tiles of 128 pixels cover 9 rows; two channel tiles: weights reloaded between runs
    (5, 64, 7, 7, 64),        # a whole image is less than half a tile
    (1, 64, 28, 28, 192),     # three channel tiles
    (4, 32, 60, 61, 64),      # rows wider than one copy of 64 pieces
    (2, 32, 112, 112, 32),    # rows of four copies, half a channel tile
]


@pytest.mark.parametrize("i", range(len(RESIDENT_CASES)))
def test_weight_resident_tile(oracle, i):
    n, ic, ih, iw, oc = RESIDENT_CASES[i]
    tile = lib.tile_names().index("v4_64x128res")
    k = ic * 9
    live = dict(scale_bias=2e-4, scale_z=0.02, scale_dst=float(np.float32(2e-4 * 73.9 * 73.3 * k ** 0.5 / 25.0)))
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            d = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 3, pad=1, nonline=nl, has_z=has_z, **live)
            assert lib.tile_usable(d, tile)
            check_case(oracle, d, seed=700 + i, algo=IGEMM, tile=tile, tag="resident-%d" % i)
    # batch-strided views, no bias
    d0 = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 3, pad=1, nonline="RELU", has_z=True, **live)
    ss, fs, bs, ds = _abi.conv_shapes(d0)
    d = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 3, pad=1, nonline="RELU", has_z=True, bias_mode=_abi.BIAS_NONE,
                            src_stride_n=int(np.prod(ss[1:])) + 64, dst_stride_n=int(np.prod(ds[1:])) + 32,
                            z_stride_n=int(np.prod(ds[1:])) + 96, **live)
    check_case(oracle, d, seed=720 + i, algo=IGEMM, tile=tile, tag="resident-%d-strided" % i)
    # what it does not take: other strides, paddings, filter sizes, channel counts
    for kw in (dict(stride=2), dict(pad=0), dict(f=5, pad=2), dict(ic=128), dict(ic=96)):
        dd = _abi.make_conv_desc("NCHW32", n, kw.get("ic", ic), ih, iw, oc, kw.get("f", 3), pad=kw.get("pad", 1),
                                 stride=kw.get("stride", 1), **live)
        assert not lib.tile_usable(dd, tile), kw


STREAM32_CASES = [
    # n, ic, ih, iw, oc, stride: pointwise over 32 .. 128 channels, 32-packed -- what the streaming kernel takes
    (2, 64, 56, 56, 256, 1),     # the expanding 1x1 of the first bottleneck
    (3, 32, 17, 23, 96, 1),      # odd sizes; three channel blocks: the second wave group is half empty
    (2, 128, 14, 14, 512, 1),    # four k-steps
    (5, 64, 7, 7, 64, 1),        # a block of 32 pixels straddles images
    (1, 96, 28, 28, 32, 1),      # a single channel block per wave, three k-steps
    (4, 64, 30, 31, 160, 2),     # strided (a projection shortcut), five channel blocks
    (2, 128, 28, 28, 1024, 2),   # the widest output it takes
]


@pytest.mark.parametrize("i", range(len(STREAM32_CASES)))
def test_streaming_pointwise_kernel_32_packed(oracle, i):
    n, ic, ih, iw, oc, stride = STREAM32_CASES[i]
    tile = lib.tile_names().index("pw32_stream")
    live = dict(scale_bias=2e-4, scale_z=0.02, scale_dst=float(np.float32(2e-4 * 73.9 * 73.3 * ic ** 0.5 / 25.0)))
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        for has_z in (False, True):
            d = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 1, stride=stride, nonline=nl, has_z=has_z, **live)
            assert lib.tile_usable(d, tile)
            check_case(oracle, d, seed=800 + i, algo=IGEMM, tile=tile, tag="stream32-%d" % i)
    d0 = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 1, stride=stride, nonline="RELU", has_z=True, **live)
    ss, fs, bs, ds = _abi.conv_shapes(d0)
    d = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 1, stride=stride, nonline="RELU", has_z=True, bias_mode=_abi.BIAS_NONE,
                            src_stride_n=int(np.prod(ss[1:])) + 64, dst_stride_n=int(np.prod(ds[1:])) + 32,
                            z_stride_n=int(np.prod(ds[1:])) + 96, **live)
    check_case(oracle, d, seed=820 + i, algo=IGEMM, tile=tile, tag="stream32-%d-strided" % i)
    # what it does not take: a filter window, more than 128 input channels, more than 1024 output channels
    for kw in (dict(f=3, pad=1), dict(ic=256), dict(oc=2048)):
        dd = _abi.make_conv_desc("NCHW32", n, kw.get("ic", ic), ih, iw, kw.get("oc", oc), kw.get("f", 1), pad=kw.get("pad", 0), **live)
        assert not lib.tile_usable(dd, tile), kw


def test_first_layer_kernel_on_random_shapes(oracle):
    """Thirty seeded random first-layer problems: every filter height and width up to 8, both strides, paddings up to
    the filter size, odd image sizes, channel counts that end inside a channel tile, every activation, with and without
    a residual -- against the checker, with scales that keep most outputs inside the int8 range."""
    rng = np.random.RandomState(2024)
    ran = 0
    for i in range(30):
        n = int(rng.randint(1, 4))
        fh, fw = int(rng.randint(1, 9)), int(rng.randint(1, 9))
        stride = int(rng.choice([1, 2]))
        pad_h, pad_w = int(rng.randint(0, fh + 1)), int(rng.randint(0, fw + 1))
        ih, iw = int(rng.randint(max(fh - 2 * pad_h, 1), 45)), int(rng.randint(max(fw - 2 * pad_w, 1), 45))
        oc = 4 * int(rng.randint(1, 50))
        nl = ["IDENTITY", "RELU", "H_SWISH"][int(rng.randint(0, 3))]
        has_z = bool(rng.randint(0, 2))
        k = 4 * fh * fw
        d = _abi.make_conv_desc("NCHW4", n, 4, ih, iw, oc, fh, fw, stride=stride, pad=(pad_h, pad_w), nonline=nl, has_z=has_z,
                                scale_bias=2e-4, scale_z=0.02, scale_dst=float(np.float32(2e-4 * 73.9 * 73.3 * k ** 0.5 / 25.0)))
        a, _ = ops.conv_bias_query(d)
        if a.id != C4:
            continue
        check_case(oracle, d, seed=900 + i, tag="c4-random-%d" % i)
        ran += 1
    assert ran >= 25


def test_profile_entry_point(oracle):
    """the timed trial run of a fast-run chooser: times one algorithm, leaves the right result in dst"""
    d = _abi.make_conv_desc("NCHW32", 8, 128, 14, 14, 128, 3, pad=1, nonline="RELU", **S)
    src, flt, bias, z = util.make_tensors(d, seed=91)
    want = oracle.conv_bias(d, src, flt, bias, z)
    ts, tf, tb = to_dev(src), to_dev(flt), to_dev(bias)
    dst = torch.zeros(_abi.conv_shapes(d)[3], dtype=torch.int8, device="cuda")
    times = {}
    for algo_id in (DIRECT, IGEMM):
        a, _ = ops.conv_bias_query(d, algo_id)
        dst.zero_()
        us = ops.conv_bias_profile(d, ts, tf, tb, None, dst, a, warmup=1, iters=5)
        say("profile", algo_id, "%.2f us" % us)
        assert 0.5 < us < 1e5
        assert np.array_equal(dst.cpu().numpy(), want)
        times[algo_id] = us
    assert times[IGEMM] < times[DIRECT]       # the MFMA kernel must beat one-thread-per-output
    from megengine_amd.lib import Mi355Error
    a, _ = ops.conv_bias_query(d, IGEMM)
    with pytest.raises(Mi355Error):
        ops.conv_bias_profile(d, ts, tf, tb, None, dst, a, warmup=0, iters=0)


def test_random_descriptors_every_kernel_family(oracle):
    """Seeded random descriptors (formats, channel counts that leave ragged tiles, filter sizes, strides, paddings,
    residual, activation): MFMA tiles drawn at random and the heuristic against the generic kernel, bit for bit; the
    generic kernel itself against the CPU checker on every fifth case."""
    import random
    rnd = random.Random(2025)
    names = lib.tile_names()
    for it in range(120):
        fmt = rnd.choice(["NCHW32", "NCHW32", "NCHW32", "NCHW32_NCHW4", "NCHW4", "NCHW4_NCHW32"])
        pin = 32 if fmt.startswith("NCHW32") else 4
        pout = 32 if fmt in ("NCHW32", "NCHW4_NCHW32") else 4
        n = rnd.randint(1, 9)
        ic = rnd.choice([32, 64, 96, 128, 256, 512]) if pin == 32 else rnd.choice([4, 8, 16, 32, 64])
        f = rnd.choice([1, 1, 3, 3, 5])
        s = rnd.choice([1, 1, 2])
        pad = rnd.randint(0, f // 2 + (1 if f > 1 else 0))
        ih = rnd.randint(max(f - 2 * pad, 1) + 1, 40)
        iw = rnd.randint(max(f - 2 * pad, 1) + 1, 40)
        oc = rnd.randint(1, 20) * 32 if pout == 32 else rnd.randint(1, 80) * 4
        has_z = rnd.random() < 0.5 and fmt in ("NCHW32", "NCHW4")
        nl = rnd.choice(["IDENTITY", "RELU", "H_SWISH"])
        d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, pad=pad, stride=s, nonline=nl, has_z=has_z,
                                scale_bias=rnd.choice([2e-4, 3.3e-5, 1e-3]), scale_z=rnd.choice([0.05, 0.013]),
                                scale_dst=rnd.choice([0.05, 0.021, 0.2]))
        say("random case", it, fmt, "n", n, "ic", ic, "hw", ih, iw, "oc", oc, "f", f, "s", s, "pad", pad, "z", has_z, nl)
        src, flt, bias, z = util.make_tensors(d, seed=300 + it, bias_range=(-20000, 20000))
        ts, tf, tb, tz = to_dev(src), to_dev(flt), to_dev(bias), to_dev(z)
        ref = ops.conv_bias_exec(d, ts, tf, tb, tz, algo=DIRECT)
        if it % 5 == 0:
            torch.cuda.synchronize()
            assert np.array_equal(ref.cpu().numpy(), oracle.conv_bias(d, src, flt, bias, z))
        usable = [t for t in range(len(names)) if lib.tile_usable(d, t)]
        for tile in rnd.sample(usable, min(4, len(usable))) + [None]:
            a, _ = ops.conv_bias_query(d, IGEMM)
            if tile is not None:
                a.tile_cfg = tile
            out = ops.conv_bias_exec(d, ts, tf, tb, tz, algo=a)
            torch.cuda.synchronize()
            assert torch.equal(out, ref), "tile %s" % (names[tile] if tile is not None else "heuristic")


# ---------------------------------------------------------------------------------------------
# the one-instruction (linear) epilogue form in every kernel family that carries it
# ---------------------------------------------------------------------------------------------

# scale pairs for which the library has a proved linear form (asserted below, so the test cannot pass vacuously);
# accumulator ranges are chosen so that the outputs cover every int8 value and both clamps
LIN_SCALES = [(1.3e-3, 0.0271), (0.5, 1.0), (1e-3, 1.0)]

LIN_CASES = [
    # tag, expected algorithm, descriptor arguments
    ("dma 1x1", IGEMM, dict(fmt="NCHW32", n=2, ic=64, ih=9, iw=7, oc=96, fh=1)),
    ("dma 3x3", IGEMM, dict(fmt="NCHW32", n=2, ic=64, ih=9, iw=11, oc=64, fh=3, pad=1)),
    ("staged nchw4", IGEMM, dict(fmt="NCHW4", n=2, ic=24, ih=9, iw=9, oc=48, fh=3, pad=1)),
    ("mixed 4->32", IGEMM, dict(fmt="NCHW4_NCHW32", n=2, ic=16, ih=8, iw=8, oc=64, fh=3, pad=1)),
    ("first layer", C4, dict(fmt="NCHW4", n=2, ic=4, ih=30, iw=30, oc=64, fh=7, pad=3, stride=2)),
    ("dw3x3 s1", DW, dict(fmt="NCHW4", n=2, ic=32, ih=14, iw=14, oc=32, fh=3, pad=1, group=32)),
    ("dw3x3 s2", DW, dict(fmt="NCHW4", n=2, ic=24, ih=15, iw=13, oc=24, fh=3, pad=1, stride=2, group=24)),
    ("dw 5x5", DW, dict(fmt="NCHW4", n=1, ic=8, ih=12, iw=12, oc=8, fh=5, pad=2, group=8)),
]


@pytest.mark.parametrize("i", range(len(LIN_CASES)))
def test_linear_epilogue_form(oracle, i):
    import ctypes as C
    tag, want_algo, c = LIN_CASES[i]
    for sb, sd in LIN_SCALES:
        for nl in ("IDENTITY", "RELU"):
            cc, dd = C.c_float(), C.c_float()
            assert lib.lib().mi355_epilogue_linear_form(sb, sd, getattr(_abi, "NL_" + nl), C.byref(cc), C.byref(dd)) == 1
            d = mk(c, nonline=nl, scale_bias=sb, scale_dst=sd)
            assert ops.conv_bias_query(d)[0].id == want_algo
            # accumulators spread over about +-200 / (sb / sd): all 256 outputs and both saturation edges occur
            span = 200.0 * sd / sb
            taps = d.fh * d.fw * (d.ic // d.group)
            amp = int(max(1, min(127, (1.5 * span / taps ** 0.5) ** 0.5)))
            b = int(min(2 ** 30, span))
            want = check_case(oracle, d, seed=400 + i, tag="lin " + tag, src_range=(-amp, amp), flt_range=(-amp, amp),
                              bias_range=(-b, b))
            assert len(np.unique(want)) >= (100 if nl == "RELU" else 200), len(np.unique(want))


def test_pointwise_4packed_random_descriptors(oracle):
    """Seeded random 4-packed pointwise problems through the chooser (streaming kernel, LDS-direct and register-staged
    tiles): ragged channel counts and pixel counts, stride 1 or 2, every activation, with and without residual."""
    rng = np.random.RandomState(20261125)
    names = lib.tile_names()
    used = set()
    for it in range(90):
        n = int(rng.randint(1, 5)); ic = 4 * int(rng.randint(1, 60)); oc = 4 * int(rng.randint(1, 80))
        ih = int(rng.randint(1, 20)); iw = int(rng.randint(1, 20)); st = int(rng.choice([1, 1, 2]))
        nl = ("IDENTITY", "RELU", "H_SWISH")[int(rng.randint(3))]
        z = bool(rng.randint(2))
        sb = float(np.float32(np.exp(rng.uniform(np.log(1e-5), np.log(2e-3)))))
        sd = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        if it % 3 == 0:   # enough pixels for the many-tile branches of the chooser
            n *= 16; ih += 20; iw += 20
        d = _abi.make_conv_desc("NCHW4", n, ic, ih, iw, oc, 1, stride=st, nonline=nl, has_z=z, scale_bias=sb, scale_z=0.03,
                                scale_dst=sd)
        a, _ = ops.conv_bias_query(d)
        used.add(names[a.tile_cfg] if a.id == IGEMM else lib.algo_names()[a.id])
        check_case(oracle, d, seed=1000 + it, tag="pw4 random %d" % it)
    assert {"pw4_stream", "dma4_128x64x128", "dma4_64x64x128", "128x128x64"} <= used, used


def test_depthwise_random_descriptors(oracle):
    """Seeded random channel-wise 3x3 problems (stride 1 or 2, any padding up to 2, ragged widths, batch-strided views):
    interior threads load through the buffer descriptor, edge threads through pointers, both forms of the epilogue."""
    rng = np.random.RandomState(7)
    for it in range(40):
        n = int(rng.randint(1, 4)); c = 4 * int(rng.randint(1, 12))
        ih = int(rng.randint(3, 40)); iw = int(rng.randint(3, 40)); st = int(rng.choice([1, 2])); pad = int(rng.randint(0, 3))
        nl = ("IDENTITY", "RELU", "H_SWISH")[int(rng.randint(3))]
        z = bool(rng.randint(2))
        sb, sd = ((1.3e-3, 0.0271) if it % 2 else (2e-4, 0.05))   # with / without a linear epilogue form
        kw = dict(group=c, stride=st, pad=pad, nonline=nl, has_z=z, scale_bias=sb, scale_z=0.04, scale_dst=sd)
        d0 = _abi.make_conv_desc("NCHW4", n, c, ih, iw, c, 3, **kw)
        if it % 4 == 0:
            ss, fs, bs, ds = _abi.conv_shapes(d0)
            kw.update(src_stride_n=int(np.prod(ss[1:])) + 48, dst_stride_n=int(np.prod(ds[1:])) + 16,
                      z_stride_n=int(np.prod(ds[1:])) + 32)
        d = _abi.make_conv_desc("NCHW4", n, c, ih, iw, c, 3, **kw)
        assert ops.conv_bias_query(d)[0].id == DW
        check_case(oracle, d, seed=2000 + it, tag="dw random %d" % it)


IN_PLACE_CASES = [
    # fmt, n, ic, ih, iw, oc, f, stride, pad, group: one shape per kernel family and tile geometry
    ("NCHW32", 3, 64, 28, 28, 256, 1, 1, 0, 1),     # pointwise, the expanding layer of a bottleneck block
    ("NCHW32", 2, 128, 14, 14, 512, 1, 1, 0, 1),
    ("NCHW32", 2, 256, 15, 13, 160, 1, 1, 0, 1),    # odd sizes, a partial channel tile
    ("NCHW32", 2, 64, 28, 28, 64, 3, 1, 1, 1),      # 3x3 (the weight-resident and patch-staged tiles)
    ("NCHW32", 2, 256, 14, 14, 256, 3, 1, 1, 1),
    ("NCHW32", 2, 128, 28, 28, 128, 3, 2, 1, 1),
    ("NCHW4", 2, 16, 28, 28, 96, 1, 1, 0, 1),       # 4-packed pointwise
    ("NCHW4", 2, 64, 20, 20, 64, 3, 1, 1, 1),
    ("NCHW4", 2, 4, 56, 56, 64, 7, 2, 3, 1),        # the first-layer kernel
    ("NCHW4", 2, 96, 28, 28, 96, 3, 1, 1, 96),      # depthwise
    ("NCHW", 2, 8, 12, 12, 8, 3, 1, 1, 1),          # the generic kernel
]


@pytest.mark.parametrize("i", range(len(IN_PLACE_CASES)))
def test_output_may_replace_the_residual(i):
    """dst == z (same buffer, same batch stride): every kernel reads the residual of an output element in the thread
    that writes the element, before the write, so the result is that of separate buffers.  Every algorithm and every
    tile that takes the shape, against the same launch with a buffer of its own for the output."""
    fmt, n, ic, ih, iw, oc, f, stride, pad, group = IN_PLACE_CASES[i]
    k = (ic // group) * f * f
    kw = dict(scale_bias=2e-4, scale_z=0.02, scale_dst=float(np.float32(2e-4 * 73.9 * 73.3 * k ** 0.5 / 25.0)))
    ran = 0
    for nl in ("RELU", "H_SWISH"):
        d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, stride=stride, pad=pad, group=group, nonline=nl, has_z=True, **kw)
        src, flt, bias, z = (to_dev(t) for t in util.make_tensors(d, seed=900 + i))
        for algo_id in (DIRECT, IGEMM, DW, C4):
            tiles = range(len(lib.tile_names())) if algo_id == IGEMM else [None]
            for tile in tiles:
                try:
                    a, _ = ops.conv_bias_query(d, algo_id)
                except Exception:
                    break  # this algorithm does not take the problem
                if tile is not None:
                    if not lib.tile_usable(d, tile):
                        continue
                    a.tile_cfg = tile
                say("in place: case", i, nl, "algo", algo_id, "tile", tile)
                want = ops.conv_bias_exec(d, src, flt, bias, z, algo=a)
                buf = z.clone()
                got = ops.conv_bias_exec(d, src, flt, bias, buf, dst=buf, algo=a)
                torch.cuda.synchronize()
                assert got.data_ptr() == buf.data_ptr()
                assert torch.equal(got, want), (i, nl, algo_id, tile)
                ran += 1
    assert ran >= 2


def _proved_triples(n, seed):
    """scale triples (and scale_bias / scale_dst) for which the library holds a proof of the residual table form for
    both activations that have one"""
    import ctypes as C
    rng = np.random.RandomState(seed)
    proved = []
    while len(proved) < n:
        c0 = float(np.exp(rng.uniform(np.log(5e-3), np.log(0.2))))
        s_d = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        s_z = float(np.float32(s_d * rng.uniform(0.3, 1.5)))
        s_b = float(np.float32(c0 * s_d))
        c, tab = C.c_float(), (C.c_float * 256)()
        if all(lib.lib().mi355_epilogue_residual_table(s_b, s_z, s_d, nl, C.byref(c), tab) == 1
               for nl in (_abi.NL_IDENTITY, _abi.NL_RELU)):
            proved.append((s_b, s_z, s_d, c0))
    return proved


def test_residual_table_form_on_the_streaming_kernel(oracle):
    """Scale triples for which the library holds a proof of the residual table form (one fused multiply-add and a table
    read per output): the streaming kernel then runs that form, and its bytes must be the checker's.  Small operand
    ranges keep most outputs inside the int8 range, so every residual value meets most output steps."""
    tile = lib.tile_names().index("pw32_stream")
    proved = _proved_triples(4, 31)
    shapes = [(2, 64, 28, 28, 256, 1), (3, 32, 17, 23, 96, 1), (2, 128, 14, 14, 512, 1), (5, 64, 7, 7, 64, 1),
              (4, 64, 30, 31, 160, 2)]
    for i, (s_b, s_z, s_d, c0) in enumerate(proved):
        n, ic, ih, iw, oc, stride = shapes[i % len(shapes)]
        # accumulator sigma ~ 40 / c0 units: about 40 output steps
        amp = max(1, min(127, int(round((40.0 / c0 / ic ** 0.5) ** 0.5 * 1.7))))
        for nl in ("IDENTITY", "RELU"):
            d = _abi.make_conv_desc("NCHW32", n, ic, ih, iw, oc, 1, stride=stride, nonline=nl, has_z=True,
                                    scale_bias=s_b, scale_z=s_z, scale_dst=s_d)
            assert lib.tile_usable(d, tile)
            a, _ = ops.conv_bias_query(d, _abi.ALGO_HEURISTIC)
            assert a.tile_cfg == tile, "the chooser takes the streaming kernel where the table is proved"
            want = check_case(oracle, d, seed=950 + i, algo=IGEMM, tile=tile, tag="table-%d" % i, src_range=(-amp, amp),
                              flt_range=(-amp, amp), bias_range=(-50, 50))
            live = float(np.mean((want > -128) & (want < 127) & (want != 0)))
            say("table form case", i, nl, "c0 %.3g" % c0, "amp", amp, "live outputs %.2f" % live)
            assert live > 0.2
