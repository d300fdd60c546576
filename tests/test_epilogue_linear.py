"""The one-instruction ("linear") epilogue form: whenever the library claims that
floor(clamp(fma(float(sfb), c, d))) equals the requantisation contract, the claim is checked here against the
CPU checker on dense integer ranges through every output step, on the int32 extremes, and the search itself is
checked for being neither vacuous (it must find a form for ordinary scales) nor over-eager (scales whose steps
lie outside the exactly convertible integers must be refused).  Host code only: no GPU needed."""
import ctypes as C
import ctypes.util

import numpy as np
import pytest

from megengine_amd import _abi, lib

_libm = C.CDLL(ctypes.util.find_library("m"))
_libm.fmaf.restype = C.c_float
_libm.fmaf.argtypes = [C.c_float, C.c_float, C.c_float]


def linear_form(s_b, s_d, nl):
    c, d = C.c_float(), C.c_float()
    r = lib.lib().mi355_epilogue_linear_form(s_b, s_d, nl, C.byref(c), C.byref(d))
    assert r in (0, 1), r
    return r == 1, np.float32(c.value), np.float32(d.value)


def eval_linear(t, c, d, relu):
    """floor(min(max(fma(float(t), c, d), lo), 127.5)) with the fma rounded once to binary32.  The fma is evaluated
    in binary64 (error < 1e-13 here) and re-done with libm's fmaf wherever that error could change the result."""
    lo = np.float32(0.0 if relu else -128.0)
    tf = t.astype(np.float32).astype(np.float64)
    y = tf * np.float64(c) + np.float64(d)

    def fin(v):
        x = v.astype(np.float32)
        return np.floor(np.minimum(np.maximum(x, lo), np.float32(127.5))).astype(np.int32)

    out = fin(y)
    eps = 1e-9 * np.maximum(1.0, np.abs(y))
    shaky = np.nonzero((fin(y - eps) != out) | (fin(y + eps) != out))[0]
    assert shaky.size < 100000
    for i in shaky:
        x = np.float32(_libm.fmaf(float(np.float32(tf[i])), float(c), float(d)))
        out[i] = int(np.floor(min(max(x, lo), np.float32(127.5))))
    return out.astype(np.int8)


def sweep_points(s_b, s_d):
    """contiguous integers through every output step (thinned between the steps when the range is long)"""
    c = float(s_b) / float(s_d)
    span = int(min(2 ** 24 + 8, 140.0 / c + 8))
    if 2 * span + 1 <= (1 << 22):
        x = np.arange(-span, span + 1, dtype=np.int64)
    else:
        ks = np.arange(-128, 129, dtype=np.float64) - 0.5
        centers = np.clip(np.round(ks / c), -span, span).astype(np.int64)
        win = np.arange(-96, 97, dtype=np.int64)
        x = np.unique(np.concatenate([(centers[:, None] + win[None, :]).ravel(),
                                      np.arange(-span, span + 1, max(1, span // (1 << 20)), dtype=np.int64)]))
    ext = np.array([-2 ** 31, -2 ** 31 + 1, -2 ** 30, -2 ** 24 - 1, -2 ** 24, 2 ** 24, 2 ** 24 + 1, 2 ** 30, 2 ** 31 - 129,
                    2 ** 31 - 1], dtype=np.int64)
    return np.unique(np.concatenate([x, ext])).astype(np.int32)


FIXED = [(0.5, 1.0), (0.25, 2.0), (0.125, 0.25), (2e-4, 0.05), (float(np.float32(0.02) * np.float32(0.01)), 0.05),
         (1.3e-3, 0.0271), (7.7e-5, 3.3e-3), (1.0, 1.0), (2.5, 1.0), (3.0, 0.7), (1e-3, 1.0)]


def random_scales(n, seed):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(n):
        s = [float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2))))) for _ in range(3)]
        out.append((float(np.float32(s[0]) * np.float32(s[1])), s[2]))
    return out


def test_claimed_forms_equal_the_contract(oracle):
    found = {0: 0, 1: 0}
    cases = FIXED + random_scales(60, 7)
    for s_b, s_d in cases:
        x = sweep_points(s_b, s_d)
        for nl in (_abi.NL_IDENTITY, _abi.NL_RELU):
            ok, c, d = linear_form(s_b, s_d, nl)
            if not ok:
                continue
            found[nl] += 1
            assert c > 0
            want = oracle.requant(x, s_b, s_d, nl)
            got = eval_linear(x, c, d, nl == _abi.NL_RELU)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "scales %r nl %d c %r d %r: x=%d linear %d contract %d" % (
                (s_b, s_d), nl, c, d, x[bad[0]], got[bad[0]], want[bad[0]])
    # the search must not be vacuous: most ordinary scale pairs have a form
    assert found[_abi.NL_RELU] >= 0.8 * len(cases), found
    assert found[_abi.NL_IDENTITY] >= 0.6 * len(cases), found


def test_refuses_what_it_cannot_prove():
    # the steps of these lie beyond +-2^24, where float(sfb) is no longer every integer
    for s_b, s_d in ((1e-9, 1.0), (1e-6, 0.5), (2 ** -30, 2 ** -4)):
        for nl in (_abi.NL_IDENTITY, _abi.NL_RELU):
            ok, _, _ = linear_form(s_b, s_d, nl)
            assert not ok, (s_b, s_d, nl)
    # scales outside the range of the multi-step fast form
    assert not linear_form(1e-30, 1.0, _abi.NL_RELU)[0]
    assert not linear_form(1.0, 1e30, _abi.NL_RELU)[0]
    c, d = C.c_float(), C.c_float()
    assert lib.lib().mi355_epilogue_linear_form(1.0, 1.0, _abi.NL_H_SWISH, C.byref(c), C.byref(d)) < 0
    assert lib.lib().mi355_epilogue_linear_form(1.0, 1.0, _abi.NL_RELU, None, C.byref(d)) < 0


def test_repeated_queries_agree():
    # answers come from a small cache: same scales, same answer, also after other scales displaced the entry
    first = [linear_form(s_b, s_d, _abi.NL_RELU) for s_b, s_d in FIXED]
    for s_b, s_d in random_scales(600, 11):
        linear_form(s_b, s_d, _abi.NL_RELU)
    again = [linear_form(s_b, s_d, _abi.NL_RELU) for s_b, s_d in FIXED]
    assert first == again
