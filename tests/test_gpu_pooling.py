"""QuantizedS8 Pooling through the C ABI against the CPU checker, bit for bit: every mode and layout over windows,
strides and paddings (incl. windows that hang over every border), the extreme values, tie-heavy inputs for the rounded
means, the ResNet stem pool and the global average pool at full size, and the reference's error for a window that
lies in the padding."""
import numpy as np
import pytest
import torch

from megengine_amd import _abi, ops
from megengine_amd.lib import Mi355Error
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

MODES = ("MAX", "AVERAGE", "AVERAGE_COUNT_EXCLUDE_PADDING")
FORMATS = (("NCHW", 1), ("NCHW4", 4), ("NCHW44", 4), ("NCHW32", 32))


def run_case(oracle, mode, fmt, n, c, ih, iw, window, stride, pad, x):
    d = _abi.make_pooling_desc(mode, fmt, n, c, ih, iw, window, stride, pad)
    say("pooling", mode, fmt, (n, c, ih, iw), window, stride, pad)
    got = ops.pooling_exec(d, torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    want = oracle.pooling(d, x)
    g = got.cpu().numpy()
    assert g.shape == want.shape
    if not np.array_equal(g, want):
        bad = np.argwhere(g != want)
        raise AssertionError("%d mismatches, first at %s: got %d want %d" % (
            len(bad), tuple(bad[0]), g[tuple(bad[0])], want[tuple(bad[0])]))


GEOMETRY = [
    # window, stride, pad, ih, iw
    ((3, 3), (2, 2), (1, 1), 12, 13),
    ((2, 2), (2, 2), (0, 0), 8, 10),
    ((3, 2), (1, 2), (1, 0), 7, 9),
    ((5, 5), (3, 3), (2, 2), 11, 11),
    ((7, 7), (7, 7), (0, 0), 7, 7),
    ((1, 1), (1, 1), (0, 0), 4, 5),
    ((3, 3), (1, 1), (2, 2), 6, 6),
    ((4, 6), (3, 1), (3, 5), 5, 3),      # window wider than the image: clipped on both sides at once
    ((2, 2), (3, 3), (0, 0), 10, 10),    # stride larger than the window
]


@pytest.mark.parametrize("gi", range(len(GEOMETRY)))
def test_modes_formats_geometry(oracle, gi):
    window, stride, pad, ih, iw = GEOMETRY[gi]
    rng = np.random.RandomState(100 + gi)
    for fmt, p in FORMATS:
        c = 96 if p == 32 else 20
        shape = _abi.packed_shape(fmt, 3, c, ih, iw)
        x = rng.randint(-128, 128, shape).astype(np.int8)
        x.reshape(-1)[:: 7] = -128
        x.reshape(-1)[3:: 11] = 127
        for mode in MODES:
            run_case(oracle, mode, fmt, 3, c, ih, iw, window, stride, pad, x)


def test_extremes_and_ties(oracle):
    rng = np.random.RandomState(5)
    for fmt, p in FORMATS:
        c = 32
        shape = _abi.packed_shape(fmt, 2, c, 9, 9)
        for fill in (-128, 127):
            x = np.full(shape, fill, np.int8)
            for mode in MODES:
                run_case(oracle, mode, fmt, 2, c, 9, 9, 3, 2, 1, x)
        # small values: window sums land on odd multiples of half the count all the time (ties, both signs)
        x = rng.randint(-3, 4, shape).astype(np.int8)
        for mode in MODES[1:]:
            run_case(oracle, mode, fmt, 2, c, 9, 9, 2, 1, 1, x)
            run_case(oracle, mode, fmt, 2, c, 9, 9, (2, 3), 1, 0, x)


@pytest.mark.parametrize("fmt", ["NCHW4", "NCHW32"])
def test_resnet_stem_pool_and_global_average_full_size(oracle, fmt):
    rng = np.random.RandomState(11)
    x = rng.randint(-128, 128, _abi.packed_shape(fmt, 64, 64, 112, 112)).astype(np.int8)
    run_case(oracle, "MAX", fmt, 64, 64, 112, 112, 3, 2, 1, x)
    x = rng.randint(-128, 128, _abi.packed_shape(fmt, 64, 2048, 7, 7)).astype(np.int8)
    for mode in MODES[1:]:
        run_case(oracle, mode, fmt, 64, 2048, 7, 7, 7, 7, 0, x)


def test_full_size_properties():
    """Size-independent properties at a size the CPU checker is not asked to redo: MAX with window 1 is the identity,
    MAX of a constant image is that constant, and the 2x2 / stride 2 mean of an image that repeats every value over
    2x2 blocks gives the values back."""
    g = torch.Generator().manual_seed(3)
    small = torch.randint(-128, 128, (128, 8, 48, 48, 32), dtype=torch.int8, generator=g)
    x = small.repeat_interleave(2, dim=2).repeat_interleave(2, dim=3).contiguous().cuda()
    d = _abi.make_pooling_desc("AVERAGE", "NCHW32", 128, 256, 96, 96, 2)
    assert torch.equal(ops.pooling_exec(d, x).cpu(), small)
    d = _abi.make_pooling_desc("MAX", "NCHW32", 128, 256, 96, 96, 2)
    assert torch.equal(ops.pooling_exec(d, x).cpu(), small)
    d = _abi.make_pooling_desc("MAX", "NCHW32", 128, 256, 96, 96, 1, 1)
    assert torch.equal(ops.pooling_exec(d, x), x)


def test_errors():
    x = torch.zeros((1, 4, 4, 4), dtype=torch.int8).cuda()
    for mode in ("MAX", "AVERAGE_COUNT_EXCLUDE_PADDING"):
        d = _abi.make_pooling_desc(mode, "NCHW", 1, 4, 4, 4, 2, 2, 2)
        with pytest.raises(Mi355Error, match="lies outside completely"):
            ops.pooling_exec(d, x)
    d = _abi.make_pooling_desc("AVERAGE", "NCHW", 1, 4, 4, 4, 2, 2, 2)
    assert torch.count_nonzero(ops.pooling_exec(d, x)) == 0
    d = _abi.make_pooling_desc("MAX", "NCHW", 1, 4, 4, 4, 5, 1, 0)        # window larger than the input
    with pytest.raises(Mi355Error):
        ops.pooling_deduce_layout(d)
    d = _abi.make_pooling_desc("MAX", _abi.FMT_NCHW4_NCHW32, 1, 4, 4, 4, 2)
    with pytest.raises(Mi355Error):
        ops.pooling_deduce_layout(d)
    d = _abi.make_pooling_desc("MAX", "NCHW32", 1, 48, 4, 4, 2)           # channels not a multiple of the pack
    with pytest.raises(Mi355Error):
        ops.pooling_deduce_layout(d)
    d = _abi.make_pooling_desc(3, "NCHW", 1, 4, 4, 4, 2)
    with pytest.raises(Mi355Error):
        ops.pooling_deduce_layout(d)
    # misaligned NCHW32 tensor
    buf = torch.zeros(1 * 32 * 4 * 4 + 16, dtype=torch.int8).cuda()
    d = _abi.make_pooling_desc("MAX", "NCHW32", 1, 32, 4, 4, 2)
    with pytest.raises(Mi355Error, match="alignment"):
        ops.pooling_exec(d, buf[4:4 + 512].view(1, 1, 4, 4, 32))
