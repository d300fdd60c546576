"""numpy-facing wrapper of the CPU parity checker (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py -- never by the megengine_amd package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from megengine_amd import _abi

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        L = C.CDLL(build())
        P = C.POINTER
        L.oracle_quantize_s8.restype = C.c_int8
        L.oracle_quantize_s8.argtypes = [C.c_float, C.c_float]
        L.oracle_quantize_s32.restype = C.c_int32
        L.oracle_quantize_s32.argtypes = [C.c_float, C.c_float]
        L.oracle_activation.restype = C.c_float
        L.oracle_activation.argtypes = [C.c_float, C.c_int]
        L.oracle_epilogue_s8.restype = C.c_int8
        L.oracle_epilogue_s8.argtypes = [C.c_int32, C.c_float, C.c_int, C.c_int8, C.c_float, C.c_int, C.c_float]
        L.oracle_convbias_s8_acc.restype = C.c_int
        L.oracle_convbias_s8_acc.argtypes = [P(_abi.ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.oracle_convbias_s8.restype = C.c_int
        L.oracle_convbias_s8.argtypes = [P(_abi.ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_void_p]
        L.oracle_convbias_s8_points.restype = C.c_int
        L.oracle_convbias_s8_points.argtypes = [P(_abi.ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                C.c_void_p, C.c_int64, C.c_void_p]
        L.oracle_relayout_deduce.restype = C.c_int
        L.oracle_relayout_deduce.argtypes = [P(_abi.RelayoutDesc), P(C.c_uint32), P(C.c_uint32)]
        L.oracle_relayout.restype = C.c_int
        L.oracle_relayout.argtypes = [P(_abi.RelayoutDesc), C.c_void_p, C.c_void_p]
        L.oracle_fastdiv.restype = C.c_float
        L.oracle_fastdiv.argtypes = [C.c_float] * 4
        L.oracle_fastdiv_sweep.restype = C.c_uint64
        L.oracle_fastdiv_sweep.argtypes = [C.c_float, C.c_uint32, C.c_uint32, C.c_uint64, P(C.c_float)]
        L.oracle_round_sweep.restype = C.c_uint64
        L.oracle_round_sweep.argtypes = [C.c_uint32, C.c_uint32, P(C.c_float)]
        L.oracle_pooling_s8.restype = C.c_int
        L.oracle_pooling_s8.argtypes = [P(_abi.PoolingDesc), C.c_void_p, C.c_void_p]
        L.oracle_elemwise_q.restype = C.c_int
        L.oracle_elemwise_q.argtypes = [P(_abi.ElemwiseDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.oracle_typecvt_f32_s8.restype = None
        L.oracle_typecvt_f32_s8.argtypes = [C.c_uint64, C.c_float, C.c_void_p, C.c_void_p]
        L.oracle_typecvt_s8_f32.restype = None
        L.oracle_typecvt_s8_f32.argtypes = [C.c_uint64, C.c_float, C.c_void_p, C.c_void_p]
        _LIB = L
    return _LIB


class OracleError(RuntimeError):
    def __init__(self, status):
        super().__init__("oracle status %d" % status)
        self.status = status


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def conv_bias(desc, src, flt, bias=None, z=None):
    """Full operator.  Arrays are C-contiguous numpy int8/int32 in the reference's layouts."""
    _, _, _, dshape = _abi.conv_shapes(desc)
    dt = {_abi.DT_QS8: np.int8, _abi.DT_QS32: np.int32, _abi.DT_F32: np.float32}[desc.dst_dtype]
    if desc.dst_stride_n:
        per_n = int(np.prod(dshape[1:]))
        dst = np.zeros((desc.n, desc.dst_stride_n), dtype=dt)
        st = lib().oracle_convbias_s8(C.byref(desc), _ptr(src), _ptr(flt), _ptr(bias), _ptr(z), _ptr(dst))
        if st:
            raise OracleError(st)
        return np.ascontiguousarray(dst[:, :per_n]).reshape(dshape)
    dst = np.zeros(dshape, dtype=dt)
    st = lib().oracle_convbias_s8(C.byref(desc), _ptr(src), _ptr(flt), _ptr(bias), _ptr(z), _ptr(dst))
    if st:
        raise OracleError(st)
    return dst


def conv_acc(desc, src, flt, bias=None):
    """int32 conv + bias (the reference's intermediate 'sfb' tensor) in dst layout."""
    _, _, _, dshape = _abi.conv_shapes(desc)
    sfb = np.zeros(dshape, dtype=np.int32)
    st = lib().oracle_convbias_s8_acc(C.byref(desc), _ptr(src), _ptr(flt), _ptr(bias), _ptr(sfb))
    if st:
        raise OracleError(st)
    return sfb


def conv_bias_points(desc, src, flt, bias, z, idx):
    """Operator output at the dense-dst linear indices `idx` (int64 array) only."""
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    out = np.zeros(idx.shape, dtype=np.int8)
    st = lib().oracle_convbias_s8_points(C.byref(desc), _ptr(src), _ptr(flt), _ptr(bias), _ptr(z), _ptr(idx),
                                         idx.size, _ptr(out))
    if st:
        raise OracleError(st)
    return out


def relayout_desc(mode, shape, group=1, oc=0, elem_bytes=1, scale_src=1.0, scale_dst=1.0):
    d = _abi.RelayoutDesc(mode=mode, ndim=len(shape), group=group, oc=oc, elem_bytes=elem_bytes,
                          scale_src=scale_src, scale_dst=scale_dst)
    for i, s in enumerate(shape):
        d.shape[i] = s
    return d


def relayout_deduce(d):
    nd = C.c_uint32()
    shp = (C.c_uint32 * 7)()
    st = lib().oracle_relayout_deduce(C.byref(d), C.byref(nd), shp)
    if st:
        raise OracleError(st)
    return tuple(shp[i] for i in range(nd.value))


def relayout(d, src):
    oshape = relayout_deduce(d)
    dst = np.zeros(oshape, dtype=src.dtype)
    st = lib().oracle_relayout(C.byref(d), _ptr(np.ascontiguousarray(src)), _ptr(dst))
    if st:
        raise OracleError(st)
    return dst


def requant(src, scale_src, scale_dst, nonline=0, z=None, scale_z=1.0):
    """int32 or int8 array (+ int8 z) -> int8 with the epilogue chain; nonline is the MI355_NL_* value"""
    if np.asarray(src).dtype == np.int8:
        src = np.ascontiguousarray(src)
        d = _abi.RequantDesc(nonline=nonline, has_z=int(z is not None), scale_src=scale_src, scale_z=scale_z,
                             scale_dst=scale_dst, count=src.size)
        dst = np.empty(src.shape, np.int8)
        zc = None if z is None else np.ascontiguousarray(z, dtype=np.int8)
        st = lib().oracle_requant_s8_s8(C.byref(d), _ptr(src), _ptr(zc) if zc is not None else None, _ptr(dst))
        if st:
            raise OracleError(st)
        return dst
    src = np.ascontiguousarray(src, dtype=np.int32)
    d = _abi.RequantDesc(nonline=nonline, has_z=int(z is not None), scale_src=scale_src, scale_z=scale_z,
                         scale_dst=scale_dst, count=src.size)
    dst = np.empty(src.shape, np.int8)
    zc = None if z is None else np.ascontiguousarray(z, dtype=np.int8)
    st = lib().oracle_requant_s32_s8(C.byref(d), _ptr(src), _ptr(zc) if zc is not None else None, _ptr(dst))
    if st:
        raise OracleError(st)
    return dst


def elemwise_q(mode, srcs, scales_src, scale_dst, dst_dtype=np.int8):
    """quantized elemwise mode (by Elemwise::Mode name) on one to three int8 or int32 arrays; returns dst_dtype"""
    srcs = [np.ascontiguousarray(s) for s in srcs]
    code = {np.dtype(np.int8): _abi.DT_QS8, np.dtype(np.int32): _abi.DT_QS32}
    d = _abi.make_elemwise_desc(mode, scales_src, scale_dst, srcs[0].size, code[srcs[0].dtype], code[np.dtype(dst_dtype)])
    dst = np.empty(srcs[0].shape, dst_dtype)
    p = [_ptr(s) for s in srcs] + [None] * (3 - len(srcs))
    st = lib().oracle_elemwise_q(C.byref(d), p[0], p[1], p[2], _ptr(dst))
    if st:
        raise OracleError(st)
    return dst


def pooling(d, src):
    """QuantizedS8 Pooling forward of an int8 array laid out in d.format; returns the int8 result"""
    src = np.ascontiguousarray(src, dtype=np.int8)
    assert src.shape == _abi.packed_shape(d.format, d.n, d.c, d.ih, d.iw), (src.shape, d.format)
    oh = (d.ih + 2 * d.pad_h - d.window_h) // d.stride_h + 1
    ow = (d.iw + 2 * d.pad_w - d.window_w) // d.stride_w + 1
    dst = np.zeros(_abi.packed_shape(d.format, d.n, d.c, oh, ow), np.int8)
    st = lib().oracle_pooling_s8(C.byref(d), _ptr(src), _ptr(dst))
    if st:
        raise OracleError(st)
    return dst


def typecvt(src, scale):
    """float32 array -> int8 (quantize) or int8 array -> float32 (dequantize)"""
    src = np.ascontiguousarray(src)
    if src.dtype == np.float32:
        dst = np.empty(src.shape, np.int8)
        lib().oracle_typecvt_f32_s8(src.size, scale, _ptr(src), _ptr(dst))
    else:
        assert src.dtype == np.int8
        dst = np.empty(src.shape, np.float32)
        lib().oracle_typecvt_s8_f32(src.size, scale, _ptr(src), _ptr(dst))
    return dst
