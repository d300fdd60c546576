"""RelayoutFormat kernels against the CPU checker (bit-exact), incl. the reference KATs on the GPU."""
import numpy as np
import pytest
import torch

from megengine_amd import _abi, ops
from tests import util
from tests.gpu_util import say, to_dev

pytestmark = pytest.mark.gpu

MODES = {"NCHW4_NCHW": _abi.RL_NCHW4_NCHW, "NCHW_NCHW4": _abi.RL_NCHW_NCHW4,
         "NCHW_NCHW4_WEIGHT": _abi.RL_NCHW_NCHW4_WEIGHT}


def run(mode, x, **kw):
    d = ops.relayout_desc(mode, x.shape, elem_bytes=x.dtype.itemsize, **kw)
    say("relayout mode", mode, "shape", x.shape, kw)
    out = ops.relayout_exec(d, to_dev(x))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_reference_kats_on_gpu(kats):
    for name, k in kats["relayout"].items():
        for dt in (np.int8, np.int32):
            got = run(MODES[k["mode"]], np.array(k["src"], dt).reshape(k["src_shape"]), group=k["group"], oc=k["oc"])
            assert list(got.shape) == k["dst_shape"], name
            assert got.reshape(-1).tolist() == k["dst"], name


CASES = [
    (_abi.RL_NCHW_NCHW4, (2, 16, 8, 8), {}),            # fast path (HW % 16 == 0)
    (_abi.RL_NCHW_NCHW4, (2, 10, 5, 7), {}),            # padding, generic
    (_abi.RL_NCHW_NCHW4, (1, 12, 4, 4), dict(group=3)),
    (_abi.RL_NCHW_NCHW4_IC_SMALL, (2, 3, 9, 9), {}),
    (_abi.RL_NCHW4_NCHW, (2, 4, 8, 8, 4), {}),
    (_abi.RL_NCHW4_NCHW, (2, 4, 5, 7, 4), dict(oc=14)),
    (_abi.RL_NCHW4_NCHW, (1, 4, 4, 4, 4), dict(oc=12, group=2)),
    (_abi.RL_NCHW_NCHW32, (2, 64, 8, 8), {}),           # fast path
    (_abi.RL_NCHW_NCHW32, (1, 96, 40, 40), {}),         # fast path, several pixel tiles + tail
    (_abi.RL_NCHW_NCHW32, (2, 40, 5, 5), {}),           # padding
    (_abi.RL_NCHW32_NCHW, (2, 2, 8, 8, 32), {}),
    (_abi.RL_NCHW32_NCHW, (1, 3, 40, 40, 32), {}),
    (_abi.RL_NCHW32_NCHW, (2, 2, 5, 5, 32), dict(oc=40)),
    (_abi.RL_NCHW_NCHW4_WEIGHT, (10, 7, 3, 3), {}),
    (_abi.RL_NCHW_NCHW4_WEIGHT, (3, 6, 5, 3, 3), {}),
    (_abi.RL_NCHW4_NCHW32, (2, 16, 6, 6, 4), {}),
    (_abi.RL_NCHW32_NCHW4, (2, 2, 6, 6, 32), {}),
]


@pytest.mark.parametrize("i", range(len(CASES)))
def test_relayout_vs_oracle(oracle, i):
    mode, shape, kw = CASES[i]
    x = util.uniform_int(900 + i, shape, -128, 127, np.int8)
    want = oracle.relayout(oracle.relayout_desc(mode, shape, **kw), x)
    assert np.array_equal(run(mode, x, **kw), want)
    x32 = util.uniform_int(950 + i, shape, -100000, 100000, np.int32)
    want = oracle.relayout(oracle.relayout_desc(mode, shape, elem_bytes=4, **kw), x32)
    assert np.array_equal(run(mode, x32, **kw), want)


def test_relayout_requant(oracle):
    """QuantizedS8{1.f} -> QuantizedS8{2.f} style requantising relayout (dnn/test/cuda/relayout_format.cpp:83-87)."""
    x = util.uniform_int(77, (2, 8, 8, 8), -128, 127, np.int8)
    for ss, sd in ((1.0, 2.0), (0.37, 0.11), (0.05, 0.05)):
        want = oracle.relayout(oracle.relayout_desc(_abi.RL_NCHW_NCHW4, x.shape, scale_src=ss, scale_dst=sd), x)
        assert np.array_equal(run(_abi.RL_NCHW_NCHW4, x, scale_src=ss, scale_dst=sd), want)


def test_roundtrip_full_size():
    """Tensors of the large-shape workload (config 4): NCHW -> NCHW32 -> NCHW is the identity and agrees with the
    closed-form numpy permutation."""
    for shape in ((8, 256, 64, 64), (4, 128, 80, 80)):
        x = util.uniform_int(5, shape, -128, 127, np.int8)
        say("roundtrip", shape)
        xd = to_dev(x)
        y = ops.relayout_exec(ops.relayout_desc(_abi.RL_NCHW_NCHW32, shape), xd)
        back = ops.relayout_exec(ops.relayout_desc(_abi.RL_NCHW32_NCHW, tuple(y.shape)), y)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), util.nchw_to_packed(x, 32))
        assert torch.equal(back, xd)
        y4 = ops.relayout_exec(ops.relayout_desc(_abi.RL_NCHW_NCHW4, shape), xd)
        back4 = ops.relayout_exec(ops.relayout_desc(_abi.RL_NCHW4_NCHW, tuple(y4.shape)), y4)
        torch.cuda.synchronize()
        assert np.array_equal(y4.cpu().numpy(), util.nchw_to_packed(x, 4))
        assert torch.equal(back4, xd)
