"""The divide-free quotient of the tiled kernels' requantisation (t = r y_lo; q = fma(r, y_hi, t) with y_hi = RN(1 / s_d)
and y_lo = RN(1 / s_d - y_hi)): for a set of dst scales (ordinary, tie-heavy, extreme)
this test finds EVERY rounding boundary of the literal chain  clamp(roundf(RN(r / s_d)))  by bisection over the floats,
written here independently of the library (numpy binary32 division, libm roundf), and evaluates the divide-free form
(libm fmaf = the device's fused multiply-add) on the 65 floats around each boundary, on both signs, for the generic and
the RELU tail.  A quotient that is wrong at any boundary r fails it.  Away from the boundaries a quotient at
most one ulp from the correctly rounded one cannot change the result, so this covers every float r.  The library's own
verdict (mi355_epilogue_quotient_form) must agree.  Host code only: no GPU needed."""
import ctypes as C
import ctypes.util

import numpy as np
import pytest

from megengine_amd import lib

_libm = C.CDLL(ctypes.util.find_library("m"))
_libm.fmaf.restype = C.c_float
_libm.fmaf.argtypes = [C.c_float, C.c_float, C.c_float]
_libm.roundf.restype = C.c_float
_libm.roundf.argtypes = [C.c_float]

f32 = np.float32


def bits_to_f32(b):
    return np.array([b], dtype=np.uint32).view(np.float32)[0]


def contract(r, s_d):
    v = f32(_libm.roundf(float(f32(r) / f32(s_d))))
    return int(min(max(v, f32(-128.0)), f32(127.0)))


def fast(r, y_hi, y_lo, relu):
    r = f32(r)
    t = f32(r * y_lo)
    q = f32(_libm.fmaf(float(r), float(y_hi), float(t)))
    if relu:
        q = min(max(q, f32(0.0)), f32(127.0))
        return int(np.floor(np.float64(q) + 0.5))
    q = min(max(q, f32(-128.0)), f32(127.0))
    return int(f32(q + f32(np.copysign(f32(0.49999997), q))))   # truncation toward zero


SCALES = [0.05, 0.0271, 1e-3, 5e-2, 2e-4, 1.0, 0.125, 3.0, 0.3, 7.7e-3, 1.9073486e-06, 123456.0, 2.0 ** -30, 0.049999997,
          0.1, 1.0 / 3.0]


@pytest.mark.parametrize("s_d", SCALES)
def test_quotient_equals_division_at_every_rounding_boundary(s_d):
    s_d = f32(s_d)
    y_hi = f32(f32(1.0) / s_d)
    y_lo = f32(np.float64(1.0) / np.float64(s_d) - np.float64(y_hi))
    yh, yl = C.c_float(), C.c_float()
    assert lib.lib().mi355_epilogue_quotient_form(float(s_d), C.byref(yh), C.byref(yl)) == 1
    assert f32(yh.value) == y_hi and f32(yl.value) == y_lo
    top = int(np.array([f32(130.0) * s_d], dtype=np.float32).view(np.uint32)[0])
    assert contract(bits_to_f32(top), s_d) == 127 and contract(-bits_to_f32(top), s_d) == -128
    boundaries = set()
    for k in range(1, 129):
        lo, hi = 0, top
        while hi - lo > 1:
            m = lo + (hi - lo) // 2
            if contract(-bits_to_f32(m), s_d) <= -k:
                hi = m
            else:
                lo = m
        boundaries.add(hi)
        for d in range(-32, 33):
            b = hi + d
            if b <= 0:
                continue
            m = bits_to_f32(b)
            want_neg, want_pos = contract(-m, s_d), contract(m, s_d)
            assert fast(-m, y_hi, y_lo, False) == want_neg, (k, d)
            assert fast(m, y_hi, y_lo, False) == want_pos, (k, d)
            assert fast(m, y_hi, y_lo, True) == want_pos, (k, d)
            assert fast(-m, y_hi, y_lo, True) == 0, (k, d)
    assert len(boundaries) == 128   # one boundary per output step: the bisection did not collapse


def test_quotient_form_refuses_scales_outside_the_envelope():
    yh, yl = C.c_float(), C.c_float()
    for s in (1e-20, 3e15, 0.0, -0.05, float("inf")):
        assert lib.lib().mi355_epilogue_quotient_form(s, C.byref(yh), C.byref(yl)) == 0
    assert lib.lib().mi355_epilogue_quotient_form(0.05, None, None) < 0
