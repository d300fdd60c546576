"""Stand-alone requantisation (the unfused ConvBias epilogue) against the CPU checker: dense sweeps of the int32 input
through every rounding boundary, tie-heavy scale pairs, all activations, with and without the second input, plus
scales that force the literal (IEEE divide) form.  The same arithmetic is the epilogue of every ConvBias kernel."""
import numpy as np
import pytest
import torch

from megengine_amd import _abi, ops
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

NL = {"IDENTITY": _abi.NL_IDENTITY, "RELU": _abi.NL_RELU, "H_SWISH": _abi.NL_H_SWISH}

# (scale_src, scale_dst, scale_z): the first three make x * s_src / s_dst land exactly on .5 for every odd / every
# fourth input; the others are "ordinary" float scales
SCALES = [
    (0.5, 1.0, 1.0),
    (0.25, 2.0, 0.5),
    (0.125, 0.25, 0.75),
    (2e-4, 0.05, 0.05),
    (float(np.float32(0.02) * np.float32(0.01)), 0.05, 0.04),
    (1.3e-3, 0.0271, 0.113),
    (7.7e-5, 3.3e-3, 1.9e-2),
]


def run_case(oracle, x, z, s_src, s_dst, s_z, nl):
    xt = torch.from_numpy(x).cuda()
    zt = None if z is None else torch.from_numpy(z).cuda()
    got = ops.requant_exec(xt, s_src, s_dst, nonline=nl, z=zt, scale_z=s_z)
    torch.cuda.synchronize()
    want = oracle.requant(x, s_src, s_dst, NL[nl], z=z, scale_z=s_z)
    g = got.cpu().numpy()
    if not np.array_equal(g, want):
        bad = np.nonzero(g != want)[0]
        raise AssertionError("%d mismatches, first: x=%d z=%s got %d want %d (scales %r %r %r, %s)" % (
            len(bad), x[bad[0]], None if z is None else z[bad[0]], g[bad[0]], want[bad[0]], s_src, s_dst, s_z, nl))


@pytest.mark.parametrize("si", range(len(SCALES)))
def test_dense_sweep_through_every_boundary(oracle, si):
    s_src, s_dst, s_z = SCALES[si]
    # inputs whose quotient covers [-140, 140]: every output value and both saturation edges, contiguous integers
    span = int(min(2 ** 23, 140.0 * s_dst / s_src))
    x = np.arange(-span, span + 1, dtype=np.int32)
    if x.size > (1 << 22):   # thin out very long ranges but keep a contiguous window around each boundary
        step = x.size // (1 << 22) + 1
        x = np.unique(np.concatenate([x[::step], np.arange(-4096, 4097, dtype=np.int32)]))
    rng = np.random.RandomState(si)
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        say("requant sweep", SCALES[si], nl, x.size)
        run_case(oracle, x, None, s_src, s_dst, s_z, nl)
        z = rng.randint(-128, 128, x.size).astype(np.int8)
        run_case(oracle, x, z, s_src, s_dst, s_z, nl)


def test_full_range_inputs_and_tail(oracle):
    rng = np.random.RandomState(9)
    for n in (1, 3, 4, 5, 1023, 65537):     # count % 4 != 0: the scalar tail
        x = rng.randint(-2 ** 31, 2 ** 31 - 1, n, dtype=np.int64).astype(np.int32)
        z = rng.randint(-128, 128, n).astype(np.int8)
        for nl in ("IDENTITY", "RELU", "H_SWISH"):
            run_case(oracle, x, z, 3.1e-9, 0.043, 0.07, nl)
            run_case(oracle, x, None, 1.0, 1.0, 1.0, nl)


def test_literal_form_scales(oracle):
    """scales outside the range of the divide-free form take the IEEE divide path"""
    rng = np.random.RandomState(4)
    x = rng.randint(-100000, 100000, 100003).astype(np.int32)
    z = rng.randint(-128, 128, x.size).astype(np.int8)
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        run_case(oracle, x, z, 1e-20, 1e-17, 3e-16, nl)
        run_case(oracle, x, None, 1e-20, 1e-17, 1.0, nl)


def test_rejects_bad_arguments():
    from megengine_amd.lib import Mi355Error
    x = torch.zeros(16, dtype=torch.int32, device="cuda")
    with pytest.raises(Mi355Error):
        ops.requant_exec(x, 1.0, 1.0, nonline="SIGMOID")
    with pytest.raises(Mi355Error):
        ops.requant_exec(x[1:], 1.0, 1.0)     # misaligned int32 view


@pytest.mark.parametrize("si", range(len(SCALES)))
def test_int8_binary_modes_exhaustive(oracle, si):
    """QADD / QFUSE_ADD_RELU / QFUSE_ADD_H_SWISH on two int8 tensors: every one of the 65536 operand pairs."""
    s_a, s_dst, s_b = SCALES[si]
    s_a = s_a * 64.0          # int8 operands: bring the quotient range to a few hundred again
    a = np.repeat(np.arange(-128, 128, dtype=np.int16), 256).astype(np.int8)
    b = np.tile(np.arange(-128, 128, dtype=np.int16), 256).astype(np.int8)
    for nl in ("IDENTITY", "RELU", "H_SWISH"):
        say("int8 pairs", (s_a, s_b, s_dst), nl)
        run_case(oracle, a, b, s_a, s_dst, s_b, nl)
        run_case(oracle, a, None, s_a, s_dst, s_b, nl)    # unary QRELU / QH_SWISH / rescaling TypeCvt


def test_int8_tail_and_alignment(oracle):
    from megengine_amd.lib import Mi355Error
    rng = np.random.RandomState(3)
    for n in (1, 15, 16, 17, 4099):
        a = rng.randint(-128, 128, n).astype(np.int8)
        b = rng.randint(-128, 128, n).astype(np.int8)
        run_case(oracle, a, b, 0.031, 0.047, 0.022, "RELU")
    x = torch.zeros(64, dtype=torch.int8, device="cuda")
    with pytest.raises(Mi355Error):
        ops.requant_exec(x[1:33], 1.0, 1.0)


def test_typecvt_float32_to_int8_and_back(oracle):
    """TypeCvt Float32 <-> QuantizedS8: dense sweeps through every rounding boundary, random bit patterns (NaN,
    infinities, denormals included), ragged lengths, and the round trip."""
    rng = np.random.RandomState(21)
    for scale in (1.0, 0.25, 0.037, 3.3e-3, 17.5):
        s = np.float32(scale)
        x = (np.arange(-140 * 4096, 140 * 4096 + 1, dtype=np.float32) / np.float32(4096)) * s
        bits = rng.randint(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
        for arr in (x, bits, x[:1], x[:5], x[:1023]):
            say("typecvt f32->s8", scale, arr.size)
            got = ops.typecvt_exec(torch.from_numpy(arr).cuda(), scale)
            torch.cuda.synchronize()
            want = oracle.typecvt(arr, scale)
            g = got.cpu().numpy()
            if not np.array_equal(g, want):
                bad = np.nonzero(g != want)[0]
                raise AssertionError("%d mismatches, first: x=%r got %d want %d (scale %r)" % (
                    len(bad), arr[bad[0]], g[bad[0]], want[bad[0]], scale))
        q = rng.randint(-128, 128, 100003).astype(np.int8)
        f = ops.typecvt_exec(torch.from_numpy(q).cuda(), scale)
        assert np.array_equal(f.cpu().numpy(), oracle.typecvt(q, scale))
        assert np.array_equal(ops.typecvt_exec(f, scale).cpu().numpy(), q)
    from megengine_amd.lib import Mi355Error
    buf = torch.zeros(64, dtype=torch.float32).cuda()
    with pytest.raises(Mi355Error, match="alignment"):
        ops.typecvt_exec(buf[1:33], 1.0)


def test_linear_form_on_every_int32():
    """The one-instruction form against the multi-step form on ALL 2^32 inputs, on the device: an all-zero second
    input forces the multi-step form (r + 0.0 is exact, so it computes the same function), which the sweeps above pin
    to the CPU checker."""
    import ctypes as C
    from megengine_amd import lib
    chunk = 1 << 26
    base = torch.arange(chunk, dtype=torch.int64, device="cuda")
    zeros = torch.zeros(chunk, dtype=torch.int8, device="cuda")
    rng = np.random.RandomState(5)
    drawn = []
    for _ in range(10):   # scale pairs drawn the way the workloads draw them
        a, b, s_dst = (float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2))))) for _ in range(3))
        drawn.append((float(np.float32(a) * np.float32(b)), s_dst))
    checked = 0
    for i, (s_src, s_dst) in enumerate([(1.3e-3, 0.0271), (0.5, 1.0), (3.1e-5, 0.011)] + drawn):
        for nl in ("IDENTITY", "RELU"):
            c, d = C.c_float(), C.c_float()
            have = lib.lib().mi355_epilogue_linear_form(s_src, s_dst, NL[nl], C.byref(c), C.byref(d))
            assert have == 1 or i >= 3, (s_src, s_dst, nl)
            if have != 1:
                continue   # no proved form for this drawn pair: the kernels run the multi-step form
            checked += 1
            say("linear form, all int32", s_src, s_dst, nl, "c", c.value, "d", d.value)
            for k in range(-(1 << 31) // chunk, (1 << 31) // chunk):
                x = (base + k * chunk).to(torch.int32)
                lin = ops.requant_exec(x, s_src, s_dst, nonline=nl)
                ref = ops.requant_exec(x, s_src, s_dst, nonline=nl, z=zeros, scale_z=0.37)
                if not torch.equal(lin, ref):
                    bad = torch.nonzero(lin != ref)[0].item()
                    raise AssertionError("x=%d: linear %d, multi-step %d (scales %r %r, %s)" % (
                        int(x[bad]), int(lin[bad]), int(ref[bad]), s_src, s_dst, nl))
    assert checked >= 18, checked


def test_stream_probe_moves_the_bytes():
    """The bench's measuring stick: reads every input vector, writes every output vector (each output is the running
    XOR of the inputs its thread has read, so an output equals its input wherever the launch gives a thread one unit)."""
    import ctypes as C
    from megengine_amd import lib
    n = 1 << 20
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
    dst = torch.zeros(n, dtype=torch.uint8, device="cuda")
    st = lib.lib().mi355_stream_probe(C.c_void_p(torch.cuda.current_stream().cuda_stream), src.data_ptr(), n, dst.data_ptr(), n)
    assert st == 0
    torch.cuda.synchronize()
    assert torch.equal(dst, src)      # 65536 units on at least as many threads: one unit per thread
    dst.zero_()
    assert lib.lib().mi355_stream_probe(C.c_void_p(torch.cuda.current_stream().cuda_stream), src.data_ptr(), n, dst.data_ptr(), n // 4) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[: n // 4], src[: n // 4]) and int(dst[n // 4:].max()) == 0
