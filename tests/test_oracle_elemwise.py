"""Pins of the checker's quantized elemwise function (oracle_elemwise_q), none of which re-types its C expressions:

* closed forms: with every scale 1 the modes are integer functions of the stored values (sum, product, max, comparison,
  a * b + c ...) clamped to the destination type -- a wrong operand order, a dropped term or a wrong comparison fails;
* the function must agree with the already pinned requantisation chain (oracle.requant) where the two overlap: ADD,
  FUSE_ADD_RELU, FUSE_ADD_H_SWISH on two QuantizedS8 tensors, RELU / H_SWISH from QuantizedS8 and QuantizedS32;
* the reference's own metamorphic test of these operators (dnn/test/naive/elemwise_multi_type.cpp:73-132, :144-225,
  :227-283: quantized mode == TypeCvt -> float Elemwise -> TypeCvt, scales 0.1 / 0.2 / 0.3 -> 0.35) restated with numpy
  float32 arrays, whose every operation rounds to binary32 on its own, and C's roundf through libm;
* QuantizedS32 destinations saturate at 2147483520 and -2147483648 (dnn/include/megdnn/dtype.h:887-896)."""
import ctypes as C
import ctypes.util

import numpy as np
import pytest

from megengine_amd import _abi

f32 = np.float32
_libm = C.CDLL(ctypes.util.find_library("m"))
_libm.roundf.restype = C.c_float
_libm.roundf.argtypes = [C.c_float]


def c_roundf(a):
    return np.array([_libm.roundf(float(v)) for v in a.ravel()], f32).reshape(a.shape)


def np_quantize(r, scale, dst_dtype):
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        v = c_roundf((r / f32(scale)).astype(f32))
    lo, hi = (-128.0, 127.0) if dst_dtype == np.int8 else (-2147483648.0, 2147483520.0)
    v = np.where(np.isnan(v), f32(lo), v)          # fmax(lo, NaN) = lo
    v = np.minimum(np.maximum(f32(lo), v), f32(hi))
    return v.astype(np.int64).astype(dst_dtype)


def np_float_kernel(mode, x, y, z):
    """the float kernels on float32 arrays (each numpy operation rounds to binary32)"""
    one, zero = f32(1), f32(0)

    def hswish(t):
        return (t * np.minimum(np.maximum(t + f32(3), zero), f32(6))) * (one / f32(6))

    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        table = {
            "RELU": lambda: np.where(x <= 0, zero, x), "ABS": lambda: np.abs(x), "CEIL": lambda: np.ceil(x),
            "FLOOR": lambda: np.floor(x), "NEGATE": lambda: -x, "ROUND": lambda: c_roundf(x),
            "FAST_TANH": lambda: (x * (f32(27) + x * x)) / (f32(27) + (f32(9) * x) * x),
            "H_SWISH": lambda: hswish(x),
            "ABS_GRAD": lambda: np.where(x > 0, y, -y), "ADD": lambda: x + y, "FLOOR_DIV": lambda: np.floor(x / y),
            "MAX": lambda: np.where(x > y, x, y), "MIN": lambda: np.where(x < y, x, y), "MUL": lambda: x * y,
            "SIGMOID_GRAD": lambda: (x * (one - x)) * y, "SUB": lambda: x - y, "SWITCH_GT0": lambda: np.where(x > 0, y, zero),
            "TANH_GRAD": lambda: (one - x * x) * y, "TRUE_DIV": lambda: x / y,
            "LT": lambda: (x < y).astype(f32), "LEQ": lambda: (x <= y).astype(f32), "EQ": lambda: (x == y).astype(f32),
            "FUSE_ADD_RELU": lambda: np.where(x + y <= 0, zero, x + y),
            "FAST_TANH_GRAD": lambda: ((((f32(-48) * (x * x)) / (f32(3) + x * x)) + f32(27)) + x * x) / ((f32(3) + x * x) * f32(9)) * y,
            "H_SWISH_GRAD": lambda: np.where(x < -3, zero, np.where(x > 3, y, ((f32(2) * x + f32(3)) / f32(6)) * y)),
            "FUSE_ADD_H_SWISH": lambda: hswish(x + y),
            "COND_LEQ_MOV": lambda: np.where(x <= y, z, zero), "COND_LT_MOV": lambda: np.where(x < y, z, zero),
            "FUSE_MUL_ADD3": lambda: x * y + z,
        }
        return table[mode]().astype(f32)


def rand_inputs(rng, arity, dtype, n):
    if dtype == np.int8:
        return [rng.randint(-128, 128, n).astype(np.int8) for _ in range(arity)]
    # QuantizedS32 values as a convolution produces them, plus the extremes
    out = []
    for _ in range(arity):
        a = rng.randint(-200000, 200001, n).astype(np.int32)
        a[:4] = [np.iinfo(np.int32).min, np.iinfo(np.int32).max, 0, -1]
        out.append(a)
    return out


@pytest.mark.parametrize("mode", sorted(_abi.EW_MODES))
def test_matches_the_references_metamorphic_chain_in_numpy_float32(oracle, mode):
    """the scales of dnn/test/naive/elemwise_multi_type.cpp (0.1, 0.2, 0.3 -> 0.35), QuantizedS8 and QuantizedS32 both ways"""
    rng = np.random.RandomState(sum(map(ord, mode)))
    arity = _abi.EW_ARITY[mode]
    for sdt, scales in ((np.int8, (0.1, 0.2, 0.3)), (np.int32, (2.5e-4, 3.5e-4, 1.5e-4)), (np.int8, (0.031, 1.7, 0.4))):
        srcs = rand_inputs(rng, arity, sdt, 6000)
        fl = [s.astype(f32) * f32(sc) for s, sc in zip(srcs, scales)] + [None] * (3 - arity)
        r = np_float_kernel(mode, *fl)
        for ddt, s_d in ((np.int8, 0.35), (np.int32, 0.35), (np.int8, 0.004)):
            got = oracle.elemwise_q(mode, srcs, scales[:arity], s_d, ddt)
            want = np_quantize(r, s_d, ddt)
            assert np.array_equal(got, want), (mode, sdt, ddt, s_d, np.argwhere(got != want)[:3])


def test_unit_scales_are_integer_functions(oracle):
    rng = np.random.RandomState(11)
    a, b, c = (rng.randint(-128, 128, 20000).astype(np.int64) for _ in range(3))
    a8, b8, c8 = (v.astype(np.int8) for v in (a, b, c))
    sat8 = lambda v: np.clip(v, -128, 127).astype(np.int8)
    one = (1.0, 1.0, 1.0)
    cases = {
        "ADD": a + b, "SUB": a - b, "MUL": a * b, "MAX": np.maximum(a, b), "MIN": np.minimum(a, b),
        "LT": (a < b) * 1, "LEQ": (a <= b) * 1, "EQ": (a == b) * 1, "FUSE_ADD_RELU": np.maximum(a + b, 0),
        "ABS_GRAD": np.where(a > 0, b, -b), "SWITCH_GT0": np.where(a > 0, b, 0),
        "TANH_GRAD": (1 - a * a) * b, "SIGMOID_GRAD": a * (1 - a) * b,
        "FUSE_MUL_ADD3": a * b + c, "COND_LEQ_MOV": np.where(a <= b, c, 0), "COND_LT_MOV": np.where(a < b, c, 0),
        "RELU": np.maximum(a, 0), "ABS": np.abs(a), "NEGATE": -a, "CEIL": a, "FLOOR": a, "ROUND": a,
    }
    for mode, want in cases.items():
        srcs = [a8, b8, c8][:_abi.EW_ARITY[mode]]
        # every intermediate is an integer below 2^24 in magnitude: float arithmetic is exact
        assert np.array_equal(oracle.elemwise_q(mode, srcs, one[:len(srcs)], 1.0, np.int32), want.astype(np.int32)), mode
        assert np.array_equal(oracle.elemwise_q(mode, srcs, one[:len(srcs)], 1.0, np.int8), sat8(want)), mode
    # an operand scale is a factor of that operand alone: a * 2 + b * 3, quantized in units of 1
    assert np.array_equal(oracle.elemwise_q("ADD", [a8, b8], (2.0, 3.0), 1.0, np.int32), (2 * a + 3 * b).astype(np.int32))
    assert np.array_equal(oracle.elemwise_q("FUSE_MUL_ADD3", [a8, b8, c8], (2.0, 3.0, 5.0), 1.0, np.int32),
                          (6 * a * b + 5 * c).astype(np.int32))
    # division: exact quotients of small integers; x / 0 saturates with the sign of x, 0 / 0 is NaN -> the lower bound
    q = oracle.elemwise_q("TRUE_DIV", [np.array([6, -6, 7, 5, -5, 0], np.int8), np.array([3, 3, 2, 0, 0, 0], np.int8)], (1.0, 1.0), 1.0)
    assert q.tolist() == [2, -2, 4, 127, -128, -128]       # 3.5 rounds away from zero
    q = oracle.elemwise_q("FLOOR_DIV", [np.array([7, -7, 6], np.int8), np.array([2, 2, -4], np.int8)], (1.0, 1.0), 1.0)
    assert q.tolist() == [3, -4, -2]


def test_overlap_with_the_requantisation_chain(oracle):
    rng = np.random.RandomState(5)
    a = rng.randint(-128, 128, 30000).astype(np.int8)
    b = rng.randint(-128, 128, 30000).astype(np.int8)
    acc = rng.randint(-300000, 300001, 30000).astype(np.int32)
    for s_a, s_b, s_d in ((0.05, 0.021, 0.04), (0.0123, 0.3, 0.11), (1.0, 1.0, 1.0)):
        for mode, nl in (("ADD", _abi.NL_IDENTITY), ("FUSE_ADD_RELU", _abi.NL_RELU), ("FUSE_ADD_H_SWISH", _abi.NL_H_SWISH)):
            assert np.array_equal(oracle.elemwise_q(mode, [a, b], (s_a, s_b), s_d),
                                  oracle.requant(a, s_a, s_d, nonline=nl, z=b, scale_z=s_b)), (mode, s_a)
        for mode, nl in (("RELU", _abi.NL_RELU), ("H_SWISH", _abi.NL_H_SWISH)):
            assert np.array_equal(oracle.elemwise_q(mode, [a], (s_a,), s_d), oracle.requant(a, s_a, s_d, nonline=nl)), mode
            assert np.array_equal(oracle.elemwise_q(mode, [acc], (s_a * 1e-3,), s_d),
                                  oracle.requant(acc, s_a * 1e-3, s_d, nonline=nl)), mode


def test_quantized_s32_destination_saturates_below_two_to_the_31(oracle):
    big = np.array([127, -128, 100, -100], np.int8)
    got = oracle.elemwise_q("MUL", [big, big], (1e6, 1e6), 1.0, np.int32)
    assert got.tolist() == [2147483520, 2147483520, 2147483520, 2147483520]
    got = oracle.elemwise_q("NEGATE", [np.array([127, -128], np.int8)], (1e9,), 1e-3, np.int32)
    assert got.tolist() == [-2147483648, 2147483520]


def test_modes_outside_the_table_are_refused(oracle):
    d = _abi.ElemwiseDesc(mode=6, arity=1, src_dtype=_abi.DT_QS8, dst_dtype=_abi.DT_QS8, scale_dst=1.0, count=1)  # EXP
    x = np.zeros(1, np.int8)
    st = oracle.lib().oracle_elemwise_q(C.byref(d), x.ctypes.data_as(C.c_void_p), None, None, x.ctypes.data_as(C.c_void_p))
    assert st == _abi.ERR_UNSUPPORTED
