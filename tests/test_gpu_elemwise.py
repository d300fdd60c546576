"""mi355_elemwise_q_exec (ElemwiseMultiType quantized modes with one to three inputs) against the CPU checker, bit for
bit: every served mode on every pairing of QuantizedS8 / QuantizedS32 inputs and destinations, ragged counts, every
pair of int8 operand values for the two-input modes, and the refusals."""
import ctypes as C

import numpy as np
import pytest
import torch

from megengine_amd import _abi, lib, ops
from tests.gpu_util import say

pytestmark = pytest.mark.gpu

TORCH = {np.dtype(np.int8): torch.int8, np.dtype(np.int32): torch.int32}


def run(oracle, mode, srcs, scales, s_d, ddt):
    got = ops.elemwise_q_exec(mode, [torch.from_numpy(s).cuda() for s in srcs], scales, s_d, dst_dtype=TORCH[np.dtype(ddt)])
    torch.cuda.synchronize()
    want = oracle.elemwise_q(mode, srcs, scales, s_d, ddt)
    g = got.cpu().numpy()
    if not np.array_equal(g, want):
        bad = np.argwhere(g != want).ravel()
        i = bad[0]
        raise AssertionError("%s: %d mismatches, first at %d: inputs %s got %d want %d (scales %r -> %r)" % (
            mode, len(bad), i, [int(s.ravel()[i]) for s in srcs], g.ravel()[i], want.ravel()[i], scales, s_d))


def inputs(rng, arity, dtype, n):
    if dtype == np.int8:
        return [rng.randint(-128, 128, n).astype(np.int8) for _ in range(arity)]
    out = []
    for _ in range(arity):
        a = rng.randint(-300000, 300001, n).astype(np.int32)
        a[:4] = [np.iinfo(np.int32).min, np.iinfo(np.int32).max, 0, -1]
        out.append(a)
    return out


@pytest.mark.parametrize("mode", sorted(_abi.EW_MODES))
def test_every_mode_and_dtype_pairing(oracle, mode):
    rng = np.random.RandomState(sum(map(ord, mode)))
    arity = _abi.EW_ARITY[mode]
    for n in (100003, 5, 4096):                      # ragged tail, fewer than one vector, whole vectors
        for sdt, scales in ((np.int8, (0.1, 0.2, 0.3)), (np.int32, (2.5e-4, 3.5e-4, 1.5e-4)), (np.int8, (0.031, 1.7, 0.4))):
            srcs = inputs(rng, arity, sdt, n)
            for ddt, s_d in ((np.int8, 0.35), (np.int32, 0.35), (np.int8, 0.004), (np.int32, 1e-6)):
                say("elemwise", mode, n, np.dtype(sdt).name, np.dtype(ddt).name, s_d)
                run(oracle, mode, srcs, scales[:arity], s_d, ddt)


@pytest.mark.parametrize("mode", sorted(m for m in _abi.EW_MODES if _abi.EW_ARITY[m] == 2))
def test_every_pair_of_int8_operands(oracle, mode):
    a, b = np.meshgrid(np.arange(-128, 128, dtype=np.int8), np.arange(-128, 128, dtype=np.int8))
    a, b = np.ascontiguousarray(a.ravel()), np.ascontiguousarray(b.ravel())
    # power-of-two scales put quotients on .5 exactly; the others are ordinary
    for scales, s_d in (((0.5, 0.25), 1.0), ((0.037, 0.052), 0.041), ((1.0, 1.0), 2.0)):
        say("elemwise pairs", mode, scales, s_d)
        run(oracle, mode, [a, b], scales, s_d, np.int8)
        run(oracle, mode, [a, b], scales, s_d * 0.01, np.int32)


def test_three_operands_on_exact_ties(oracle):
    rng = np.random.RandomState(3)
    a, b, c = (rng.randint(-128, 128, 1 << 18).astype(np.int8) for _ in range(3))
    for mode in ("FUSE_MUL_ADD3", "COND_LEQ_MOV", "COND_LT_MOV"):
        run(oracle, mode, [a, b, c], (0.5, 0.5, 0.25), 1.0, np.int8)     # a*b/4 + c/4: quarters, ties included
        run(oracle, mode, [a, b, c], (0.011, 0.017, 0.003), 1.9e-3, np.int8)


def test_refusals():
    L = lib.lib()
    x = torch.zeros(64, dtype=torch.int8, device="cuda")
    p = C.c_void_p(x.data_ptr())

    def call(d, s0=p, s1=p, s2=p, dst=p):
        return L.mi355_elemwise_q_exec(None, C.byref(d), s0, s1, s2, dst)

    d = _abi.make_elemwise_desc("ADD", (1.0, 1.0), 1.0, 64)
    assert call(d) == _abi.OK
    d.mode = 6                                      # EXP: a libm mode
    assert call(d) == _abi.ERR_UNSUPPORTED
    d = _abi.make_elemwise_desc("ADD", (1.0, 1.0), 1.0, 64)
    d.arity = 3
    assert call(d) == _abi.ERR_BAD_ARG
    d = _abi.make_elemwise_desc("ADD", (1.0, 1.0), 1.0, 64)
    assert call(d, s1=None) == _abi.ERR_BAD_ARG
    assert call(d, s0=C.c_void_p(x.data_ptr() + 1)) == _abi.ERR_BAD_ARG
    d.dst_dtype = _abi.DT_F32
    assert call(d) == _abi.ERR_UNSUPPORTED
    d = _abi.make_elemwise_desc("ADD", (1.0, 1.0), 1.0, 0)
    assert call(d, s0=None, s1=None, dst=None) == _abi.OK   # nothing to do
    torch.cuda.synchronize()
