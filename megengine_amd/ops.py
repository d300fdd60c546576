"""Host-side Python mirror of the two operators, over torch device tensors.

PyTorch is plumbing only here: it owns device memory and the stream.  All arithmetic happens in
the HIP kernels behind the C ABI; a missing library or a non-GPU tensor raises.

The calls mirror megdnn::ConvBiasForward (dnn/include/megdnn/oprs/nn.h:358-536):
    deduce_layout            -> conv_bias_deduce_layout(desc)
    get_workspace_in_bytes   -> conv_bias_workspace(desc, algo)
    get_algorithm_heuristic  -> conv_bias_query(desc)
    exec(src, filter, bias, z, dst, workspace) -> conv_bias_exec(...)
and megdnn::RelayoutFormat (dnn/include/megdnn/oprs/general.h:1348-1373); requant_exec is the unfused
epilogue (the reference's post-process pass; unary ElemwiseMultiType quantized modes and TypeCvt s32 -> s8).
"""
import ctypes as C

import torch

from . import _abi
from .lib import check, lib


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise RuntimeError("mi355 operators take GPU tensors only (got %s)" % t.device)
    if not t.is_contiguous():
        raise RuntimeError("tensor must be contiguous")
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def conv_bias_deduce_layout(desc):
    oh, ow = C.c_uint32(), C.c_uint32()
    check(lib().mi355_convbias_deduce_out(C.byref(desc), C.byref(oh), C.byref(ow)))
    return _abi.conv_shapes(desc)[3]


def conv_bias_query(desc, algo=_abi.ALGO_HEURISTIC):
    """-> (Algo, workspace_bytes)"""
    a = _abi.Algo()
    ws = C.c_size_t()
    check(lib().mi355_convbias_s8_query(C.byref(desc), algo, C.byref(a), C.byref(ws)))
    return a, ws.value


def conv_bias_workspace(desc, algo=_abi.ALGO_HEURISTIC):
    return conv_bias_query(desc, algo)[1]


def conv_bias_exec(desc, src, flt, bias=None, z=None, dst=None, algo=None, workspace=None):
    if algo is None:
        algo, ws_bytes = conv_bias_query(desc)
    elif isinstance(algo, int):
        algo, ws_bytes = conv_bias_query(desc, algo)
    else:
        ws_bytes = conv_bias_query(desc, algo.id)[1] if workspace is None and algo.id >= 0 else 0
    if dst is None:
        shape = _abi.conv_shapes(desc)[3]
        dt = {_abi.DT_QS8: torch.int8, _abi.DT_QS32: torch.int32, _abi.DT_F32: torch.float32}[desc.dst_dtype]
        if desc.dst_stride_n:
            dst = torch.empty((desc.n, desc.dst_stride_n), dtype=dt, device=src.device)
        else:
            dst = torch.empty(shape, dtype=dt, device=src.device)
    if workspace is None and ws_bytes:
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=src.device)
    wsn = workspace.numel() if workspace is not None else 0
    check(lib().mi355_convbias_s8_exec(_stream(), C.byref(desc), C.byref(algo), _ptr(src), _ptr(flt), _ptr(bias),
                                      _ptr(z), _ptr(dst), _ptr(workspace), wsn))
    return dst


def conv_bias_preprocess(desc, flt, algo):
    """exec_preprocess: the filter re-tiled for `algo` (a torch uint8 tensor), or None when the algorithm reads the
    reference layout only (deduce_preprocessed_filter_layout returns nothing for it)."""
    n = C.c_size_t()
    check(lib().mi355_convbias_s8_preprocess_size(C.byref(desc), C.byref(algo), C.byref(n)))
    if n.value == 0:
        return None
    out = torch.empty(n.value, dtype=torch.uint8, device=flt.device)
    check(lib().mi355_convbias_s8_preprocess(_stream(), C.byref(desc), C.byref(algo), _ptr(flt), _ptr(out), n.value))
    return out


def conv_bias_exec_preprocessed(desc, src, pre, bias=None, z=None, dst=None, algo=None):
    if dst is None:
        dst = torch.empty(_abi.conv_shapes(desc)[3], dtype=torch.int8, device=src.device)
    check(lib().mi355_convbias_s8_exec_preprocessed(_stream(), C.byref(desc), C.byref(algo), _ptr(src), _ptr(pre),
                                                   pre.numel(), _ptr(bias), _ptr(z), _ptr(dst), None, 0))
    return dst


def conv_bias_profile(desc, src, flt, bias, z, dst, algo, warmup=2, iters=10, workspace=None):
    """Average time in microseconds of one launch of `algo` (synchronises the current stream, overwrites dst)."""
    us = C.c_float()
    wsn = workspace.numel() if workspace is not None else 0
    check(lib().mi355_convbias_s8_profile(_stream(), C.byref(desc), C.byref(algo), _ptr(src), _ptr(flt), _ptr(bias),
                                         _ptr(z), _ptr(dst), _ptr(workspace), wsn, warmup, iters, C.byref(us)))
    return us.value


def conv_bias_bind(desc, src, flt, bias, z, dst, algo, workspace=None, stream=None, preprocessed=None):
    """Pre-marshals one exec call; the returned callable launches it on the CURRENT torch stream
    when `stream` is None, else on that raw stream handle, and raises on a non-zero status.
    Keeps the tensors alive.  For callers that replay the same launch many times.  With `preprocessed` (the result of
    conv_bias_preprocess for the same algo) the call is exec with a PreprocessedFilter."""
    wsn = workspace.numel() if workspace is not None else 0
    if preprocessed is not None:
        fn = lib().mi355_convbias_s8_exec_preprocessed
        tail = (C.byref(desc), C.byref(algo), _ptr(src), _ptr(preprocessed), preprocessed.numel(), _ptr(bias), _ptr(z),
                _ptr(dst), _ptr(workspace), wsn)
    else:
        fn = lib().mi355_convbias_s8_exec
        tail = (C.byref(desc), C.byref(algo), _ptr(src), _ptr(flt), _ptr(bias), _ptr(z), _ptr(dst), _ptr(workspace), wsn)
    keep = (desc, algo, src, flt, bias, z, dst, workspace, preprocessed)
    fixed = None if stream is None else C.c_void_p(stream)

    def call(_keep=keep):
        st = fixed if fixed is not None else C.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = fn(st, *tail)
        if rc:
            check(rc)

    return call


def relayout_desc(mode, shape, group=1, oc=0, elem_bytes=1, scale_src=1.0, scale_dst=1.0):
    d = _abi.RelayoutDesc(mode=mode, ndim=len(shape), group=group, oc=oc, elem_bytes=elem_bytes,
                          scale_src=scale_src, scale_dst=scale_dst)
    for i, s in enumerate(shape):
        d.shape[i] = s
    return d


def relayout_deduce_layout(d):
    nd = C.c_uint32()
    shp = (C.c_uint32 * 7)()
    check(lib().mi355_relayout_deduce(C.byref(d), C.byref(nd), shp))
    return tuple(shp[i] for i in range(nd.value))


def relayout_exec(d, src, dst=None):
    if dst is None:
        dst = torch.empty(relayout_deduce_layout(d), dtype=src.dtype, device=src.device)
    check(lib().mi355_relayout_exec(_stream(), C.byref(d), _ptr(src), _ptr(dst)))
    return dst


def requant_exec(src, scale_src, scale_dst, nonline="IDENTITY", z=None, scale_z=1.0, dst=None):
    """QuantizedS32 or QuantizedS8 (+ QuantizedS8 z) -> QuantizedS8 with the ConvBias epilogue arithmetic."""
    nl = nonline if isinstance(nonline, int) else {"IDENTITY": _abi.NL_IDENTITY, "RELU": _abi.NL_RELU,
                                                    "H_SWISH": _abi.NL_H_SWISH, "SIGMOID": 2}[nonline]
    if src.dtype not in (torch.int32, torch.int8):
        raise RuntimeError("requant_exec takes an int32 or int8 tensor")
    if dst is None:
        dst = torch.empty(src.shape, dtype=torch.int8, device=src.device)
    d = _abi.RequantDesc(nonline=nl, has_z=int(z is not None), scale_src=scale_src, scale_z=scale_z, scale_dst=scale_dst,
                         count=src.numel())
    fn = lib().mi355_requant_s32_s8_exec if src.dtype == torch.int32 else lib().mi355_requant_s8_s8_exec
    check(fn(_stream(), C.byref(d), _ptr(src), _ptr(z), _ptr(dst)))
    return dst


def elemwise_q_exec(mode, srcs, scales_src, scale_dst, dst_dtype=None, dst=None):
    """ElemwiseMultiType quantized mode `mode` (name of the Elemwise::Mode, e.g. "FUSE_MUL_ADD3") on one to three int8 or
    int32 tensors of one shape with their scales; dst is QuantizedS8 unless dst_dtype says torch.int32."""
    if len(srcs) != _abi.EW_ARITY[mode]:
        raise RuntimeError("%s takes %d inputs" % (mode, _abi.EW_ARITY[mode]))
    if any(s.dtype != srcs[0].dtype or s.shape != srcs[0].shape for s in srcs) or srcs[0].dtype not in (torch.int8, torch.int32):
        raise RuntimeError("elemwise_q_exec takes int8 or int32 tensors of one dtype and shape")
    ddt = torch.int8 if dst_dtype is None else dst_dtype
    if dst is None:
        dst = torch.empty(srcs[0].shape, dtype=ddt, device=srcs[0].device)
    code = {torch.int8: _abi.DT_QS8, torch.int32: _abi.DT_QS32}
    d = _abi.make_elemwise_desc(mode, scales_src, scale_dst, srcs[0].numel(), code[srcs[0].dtype], code[dst.dtype])
    p = [_ptr(s) for s in srcs] + [None] * (3 - len(srcs))
    check(lib().mi355_elemwise_q_exec(_stream(), C.byref(d), p[0], p[1], p[2], _ptr(dst)))
    return dst


def pooling_deduce_layout(d):
    """Output shape of megdnn::PoolingForward for the descriptor (dnn/src/common/pooling.cpp:7-125)."""
    oh, ow = C.c_uint32(), C.c_uint32()
    check(lib().mi355_pooling_deduce_out(C.byref(d), C.byref(oh), C.byref(ow)))
    return _abi.packed_shape(d.format, d.n, d.c, oh.value, ow.value)


def pooling_exec(d, src, dst=None):
    """megdnn::PoolingForward::exec on a QuantizedS8 tensor (dst carries the scale of src)."""
    if src.dtype != torch.int8:
        raise RuntimeError("pooling_exec takes an int8 tensor")
    if tuple(src.shape) != _abi.packed_shape(d.format, d.n, d.c, d.ih, d.iw):
        raise RuntimeError("src shape %s does not match the descriptor" % (tuple(src.shape),))
    if dst is None:
        dst = torch.empty(pooling_deduce_layout(d), dtype=torch.int8, device=src.device)
    check(lib().mi355_pooling_s8_exec(_stream(), C.byref(d), _ptr(src), _ptr(dst)))
    return dst


def typecvt_exec(src, scale, dst=None):
    """megdnn::TypeCvt between Float32 and QuantizedS8: a float32 tensor is quantized with `scale`, an int8 tensor is
    dequantized with it."""
    if src.dtype == torch.float32:
        if dst is None:
            dst = torch.empty(src.shape, dtype=torch.int8, device=src.device)
        check(lib().mi355_typecvt_f32_s8_exec(_stream(), src.numel(), scale, _ptr(src), _ptr(dst)))
    elif src.dtype == torch.int8:
        if dst is None:
            dst = torch.empty(src.shape, dtype=torch.float32, device=src.device)
        check(lib().mi355_typecvt_s8_f32_exec(_stream(), src.numel(), scale, _ptr(src), _ptr(dst)))
    else:
        raise RuntimeError("typecvt_exec takes a float32 or an int8 tensor")
    return dst
