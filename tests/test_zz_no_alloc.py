"""The allocation-free exec entry point (mi355_convbias_s8_exec_static_workspace) against mi355_convbias_s8_exec.

Collected last on purpose (the file name sorts after every other test file): the suite runs with -x, and a failure here
must not hide the tests of the operator proper."""
import ctypes as C

import numpy as np
import pytest
import torch

from megengine_amd import _abi, lib, ops
from tests import util

pytestmark = pytest.mark.gpu

S = dict(scale_bias=2e-4, scale_z=0.05, scale_dst=0.05)


def _exec_static(d, algo, src, flt, bias, z, dst):
    return lib.lib().mi355_convbias_s8_exec_static_workspace(
        C.c_void_p(torch.cuda.current_stream().cuda_stream), C.byref(d), None if algo is None else C.byref(algo), ops._ptr(src),
        ops._ptr(flt), ops._ptr(bias), ops._ptr(z), ops._ptr(dst))


def _case(d, seed):
    src, flt, bias, z = util.make_tensors(d, seed=seed)
    return [None if x is None else torch.from_numpy(x).cuda() for x in (src, flt, bias, z)]


def test_static_workspace_exec_matches_exec_two_calls_in_a_row():
    """Two calls in a row on the one array, the second with a smaller input (its tensors cover only the front of what
    the first call left behind), then the first again: each must equal mi355_convbias_s8_exec with a workspace of the
    caller's, bit for bit, for the algorithm that needs the workspace (plain NCHW through relayout + MFMA)."""
    nchw = lib.algo_names().index("MI355_NCHW_RELAYOUT_MFMA_I8")
    big = _abi.make_conv_desc("NCHW", 4, 24, 28, 28, 40, 3, pad=1, nonline="RELU", has_z=True, **S)
    small = _abi.make_conv_desc("NCHW", 2, 20, 19, 23, 36, 3, pad=1, nonline="H_SWISH", has_z=True, **S)
    assert lib.lib().mi355_static_workspace_bytes() == 32 << 20
    plans = []
    for d, seed in ((big, 5), (small, 6)):
        algo, ws = ops.conv_bias_query(d, nchw)
        assert algo.id == nchw and 0 < ws <= lib.lib().mi355_static_workspace_bytes()
        t = _case(d, seed)
        want = ops.conv_bias_exec(d, *t, algo=algo, workspace=torch.empty(ws, dtype=torch.uint8, device="cuda"))
        torch.cuda.synchronize()
        plans.append((d, algo, t, want))
    for d, algo, t, want in (plans[0], plans[1], plans[0]):
        got = torch.full_like(want, 77)
        assert _exec_static(d, algo, *t, got) == 0, lib.lib().mi355_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    # without an algorithm the heuristic makes the same choice, inside the array
    d, algo, t, want = plans[1]
    got = torch.full_like(want, 77)
    assert _exec_static(d, None, *t, got) == 0, lib.lib().mi355_last_error()
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_static_workspace_exec_runs_the_other_algorithms_unchanged():
    """Algorithms without a workspace go through the same entry point untouched."""
    d = _abi.make_conv_desc("NCHW32", 2, 64, 14, 14, 64, 3, pad=1, nonline="RELU", has_z=True, **S)
    t = _case(d, 9)
    algo, ws = ops.conv_bias_query(d)
    assert ws == 0
    want = ops.conv_bias_exec(d, *t, algo=algo)
    got = torch.full_like(want, 77)
    assert _exec_static(d, algo, *t, got) == 0, lib.lib().mi355_last_error()
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_static_workspace_exec_refuses_what_does_not_fit():
    """A problem whose workspace exceeds the array: MI355_ERR_WORKSPACE for the algorithm by name, the generic kernel from
    the heuristic; nothing is launched in the first case."""
    nchw = lib.algo_names().index("MI355_NCHW_RELAYOUT_MFMA_I8")
    d = _abi.make_conv_desc("NCHW", 32, 64, 112, 112, 64, 3, pad=1, nonline="RELU", **S)
    algo, ws = ops.conv_bias_query(d, nchw)
    assert ws > lib.lib().mi355_static_workspace_bytes()
    ss, fs, bs, ds = _abi.conv_shapes(d)
    src = torch.zeros(ss, dtype=torch.int8, device="cuda")
    flt = torch.zeros(fs, dtype=torch.int8, device="cuda")
    bias = torch.zeros(bs, dtype=torch.int32, device="cuda")
    dst = torch.full(ds, 77, dtype=torch.int8, device="cuda")
    assert _exec_static(d, algo, src, flt, bias, None, dst) == _abi.ERR_WORKSPACE
    assert "static workspace" in lib.lib().mi355_last_error().decode()
    torch.cuda.synchronize()
    assert int((dst != 77).sum()) == 0
