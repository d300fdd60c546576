"""ctypes mirror of include/mi355_convbias.h (struct layouts and enum values).

Only plain data lives here, so both the product binding (megengine_amd.lib) and the CPU
parity checker's wrapper can share one definition of the descriptors.
"""
import ctypes as C

ABI_VERSION = 1

# mi355_status
OK, ERR_BAD_ARG, ERR_UNSUPPORTED, ERR_SHAPE, ERR_WORKSPACE, ERR_LAUNCH, ERR_NO_DEVICE, ERR_ALGO = range(8)

# param::ConvBias::Format
FMT_NCHW, FMT_NCHW4, FMT_NCHW32, FMT_NCHW44, FMT_NCHW4_NCHW32, FMT_NCHW32_NCHW4, FMT_NCHW4_NCHW = 0, 3, 5, 7, 9, 10, 11
FORMAT_NAMES = {
    "NCHW": FMT_NCHW, "NCHW4": FMT_NCHW4, "NCHW32": FMT_NCHW32, "NCHW44": FMT_NCHW44,
    "NCHW4_NCHW32": FMT_NCHW4_NCHW32, "NCHW32_NCHW4": FMT_NCHW32_NCHW4, "NCHW4_NCHW": FMT_NCHW4_NCHW,
}
# param::ConvBias::NonlineMode
NL_IDENTITY, NL_RELU, NL_SIGMOID, NL_H_SWISH = 0, 1, 2, 3
NONLINE_NAMES = {"IDENTITY": NL_IDENTITY, "RELU": NL_RELU, "SIGMOID": NL_SIGMOID, "H_SWISH": NL_H_SWISH}
MODE_CROSS_CORRELATION, MODE_CONVOLUTION = 0, 1
SPARSE_DENSE, SPARSE_GROUP = 0, 1
BIAS_NONE, BIAS_BROADCAST_CHANNEL, BIAS_FULL = 0, 1, 2
DT_QS8, DT_QS32, DT_F32 = 0, 1, 2

ALGO_HEURISTIC = -1
ALGO_HEURISTIC_PREPROCESS = -2

# param::RelayoutFormat::Mode (+ extension modes 32..35)
RL_NCHW_NCHW4_IC_SMALL = 22
RL_NCHW_NCHW4 = 24
RL_NCHW4_NCHW = 25
RL_NCHW_NCHW4_WEIGHT = 26
RL_NCHW_NCHW32 = 32
RL_NCHW32_NCHW = 33
RL_NCHW4_NCHW32 = 34
RL_NCHW32_NCHW4 = 35


class ConvDesc(C.Structure):
    _fields_ = [
        ("format", C.c_uint32), ("sparse", C.c_uint32), ("nonline", C.c_uint32), ("mode", C.c_uint32),
        ("n", C.c_uint32), ("ic", C.c_uint32), ("ih", C.c_uint32), ("iw", C.c_uint32),
        ("oc", C.c_uint32), ("fh", C.c_uint32), ("fw", C.c_uint32),
        ("group", C.c_uint32),
        ("pad_h", C.c_uint32), ("pad_w", C.c_uint32), ("stride_h", C.c_uint32), ("stride_w", C.c_uint32),
        ("dilate_h", C.c_uint32), ("dilate_w", C.c_uint32),
        ("dst_dtype", C.c_uint32), ("bias_mode", C.c_uint32), ("has_z", C.c_uint32),
        ("scale_bias", C.c_float), ("scale_z", C.c_float), ("scale_dst", C.c_float),
        ("src_stride_n", C.c_int64), ("dst_stride_n", C.c_int64), ("z_stride_n", C.c_int64),
    ]

    def key(self):
        return tuple(getattr(self, f) for f, _ in self._fields_)


class Algo(C.Structure):
    _fields_ = [("id", C.c_int32), ("tile_cfg", C.c_int32), ("reserved", C.c_uint64)]


class DeviceInfo(C.Structure):
    _fields_ = [
        ("device", C.c_int32), ("compute_units", C.c_int32), ("clock_khz", C.c_int32),
        ("lds_bytes_per_cu", C.c_int32), ("hbm_bytes", C.c_int64),
        ("arch", C.c_char * 32), ("name", C.c_char * 96),
    ]


class RelayoutDesc(C.Structure):
    _fields_ = [
        ("mode", C.c_uint32), ("ndim", C.c_uint32), ("shape", C.c_uint32 * 7),
        ("group", C.c_uint32), ("oc", C.c_uint32), ("elem_bytes", C.c_uint32),
        ("scale_src", C.c_float), ("scale_dst", C.c_float),
    ]


class RequantDesc(C.Structure):
    _fields_ = [
        ("nonline", C.c_uint32), ("has_z", C.c_uint32), ("scale_src", C.c_float), ("scale_z", C.c_float),
        ("scale_dst", C.c_float), ("reserved", C.c_uint32), ("count", C.c_uint64),
    ]


# param::Elemwise::Mode values of the quantized modes that mi355_elemwise_q_exec serves (dnn/scripts/opr_param_defs.py:341-455)
EW_MODES = {
    "RELU": 0, "ABS": 1, "CEIL": 4, "FLOOR": 8, "NEGATE": 11, "ABS_GRAD": 15, "ADD": 16, "FLOOR_DIV": 17, "MAX": 18,
    "MIN": 19, "MUL": 21, "SIGMOID_GRAD": 23, "SUB": 24, "SWITCH_GT0": 25, "TANH_GRAD": 26, "TRUE_DIV": 27, "LT": 29,
    "LEQ": 30, "EQ": 31, "COND_LEQ_MOV": 34, "FUSE_MUL_ADD3": 35, "FUSE_ADD_RELU": 37, "FAST_TANH": 40,
    "FAST_TANH_GRAD": 41, "ROUND": 42, "H_SWISH": 49, "H_SWISH_GRAD": 50, "FUSE_ADD_H_SWISH": 51, "COND_LT_MOV": 60,
}
EW_ARITY = {m: 1 for m in ("RELU", "ABS", "CEIL", "FLOOR", "NEGATE", "ROUND", "FAST_TANH", "H_SWISH")}
EW_ARITY.update({m: 3 for m in ("COND_LEQ_MOV", "COND_LT_MOV", "FUSE_MUL_ADD3")})
EW_ARITY.update({m: 2 for m in EW_MODES if m not in EW_ARITY})


class ElemwiseDesc(C.Structure):
    _fields_ = [
        ("mode", C.c_uint32), ("arity", C.c_uint32), ("src_dtype", C.c_uint32), ("dst_dtype", C.c_uint32),
        ("scale_src", C.c_float * 3), ("scale_dst", C.c_float), ("count", C.c_uint64),
    ]


def make_elemwise_desc(mode, scales_src, scale_dst, count, src_dtype=None, dst_dtype=None):
    """mode by name; scales_src holds one scale per input of the mode"""
    d = ElemwiseDesc(mode=EW_MODES[mode], arity=EW_ARITY[mode], src_dtype=DT_QS8 if src_dtype is None else src_dtype,
                     dst_dtype=DT_QS8 if dst_dtype is None else dst_dtype, scale_dst=scale_dst, count=count)
    assert len(scales_src) == EW_ARITY[mode]
    for i, s in enumerate(scales_src):
        d.scale_src[i] = s
    return d


# param::Pooling::Mode
POOL_MAX, POOL_AVERAGE, POOL_AVERAGE_COUNT_EXCLUDE_PADDING = 0, 1, 2
POOL_NAMES = {"MAX": POOL_MAX, "AVERAGE": POOL_AVERAGE, "AVERAGE_COUNT_EXCLUDE_PADDING": POOL_AVERAGE_COUNT_EXCLUDE_PADDING}


class PoolingDesc(C.Structure):
    _fields_ = [
        ("mode", C.c_uint32), ("format", C.c_uint32),
        ("n", C.c_uint32), ("c", C.c_uint32), ("ih", C.c_uint32), ("iw", C.c_uint32),
        ("pad_h", C.c_uint32), ("pad_w", C.c_uint32), ("stride_h", C.c_uint32), ("stride_w", C.c_uint32),
        ("window_h", C.c_uint32), ("window_w", C.c_uint32),
    ]


def make_pooling_desc(mode, fmt, n, c, ih, iw, window, stride=None, pad=0):
    """window / stride / pad: an int or an (h, w) pair; stride defaults to the window (param::Pooling defaults are 2, 2)."""
    two = lambda v: (v, v) if isinstance(v, int) else tuple(v)
    wh, ww = two(window)
    sh, sw = two(window if stride is None else stride)
    ph, pw = two(pad)
    return PoolingDesc(mode=POOL_NAMES.get(mode, mode), format=FORMAT_NAMES.get(fmt, fmt), n=n, c=c, ih=ih, iw=iw,
                       pad_h=ph, pad_w=pw, stride_h=sh, stride_w=sw, window_h=wh, window_w=ww)


def packed_shape(fmt, n, c, h, w):
    """Tensor shape of (n, c, h, w) activations in a ConvBias / Pooling format."""
    p = {FMT_NCHW: 1, FMT_NCHW4: 4, FMT_NCHW44: 4, FMT_NCHW32: 32}[FORMAT_NAMES.get(fmt, fmt)]
    return (n, c, h, w) if p == 1 else (n, c // p, h, w, p)


def in_pack(fmt):
    return {FMT_NCHW: 1, FMT_NCHW4: 4, FMT_NCHW44: 4, FMT_NCHW4_NCHW32: 4, FMT_NCHW4_NCHW: 4}.get(fmt, 32)


def out_pack(fmt):
    return {FMT_NCHW: 1, FMT_NCHW4_NCHW: 1, FMT_NCHW4: 4, FMT_NCHW44: 4, FMT_NCHW32_NCHW4: 4}.get(fmt, 32)


def out_size(i, f, d, s, p):
    """infer_conv_shape (dnn/src/common/utils.cpp:130-138)."""
    return (i + 2 * p - ((f - 1) * d + 1)) // s + 1


def make_conv_desc(fmt, n, ic, ih, iw, oc, fh, fw=None, *, group=1, pad=0, stride=1, dilate=1,
                   nonline=NL_IDENTITY, mode=MODE_CROSS_CORRELATION, bias_mode=BIAS_BROADCAST_CHANNEL,
                   has_z=False, scale_bias=1.0, scale_z=1.0, scale_dst=1.0, dst_dtype=DT_QS8,
                   src_stride_n=0, dst_stride_n=0, z_stride_n=0):
    if isinstance(fmt, str):
        fmt = FORMAT_NAMES[fmt]
    if isinstance(nonline, str):
        nonline = NONLINE_NAMES[nonline]
    fw = fh if fw is None else fw
    ph, pw = (pad, pad) if isinstance(pad, int) else pad
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    dh, dw = (dilate, dilate) if isinstance(dilate, int) else dilate
    return ConvDesc(
        format=fmt, sparse=SPARSE_GROUP if group > 1 else SPARSE_DENSE, nonline=nonline, mode=mode,
        n=n, ic=ic, ih=ih, iw=iw, oc=oc, fh=fh, fw=fw, group=group,
        pad_h=ph, pad_w=pw, stride_h=sh, stride_w=sw, dilate_h=dh, dilate_w=dw,
        dst_dtype=dst_dtype, bias_mode=bias_mode, has_z=1 if has_z else 0,
        scale_bias=scale_bias, scale_z=scale_z, scale_dst=scale_dst,
        src_stride_n=src_stride_n, dst_stride_n=dst_stride_n, z_stride_n=z_stride_n)


def conv_shapes(d):
    """(src, filter, bias, dst) shapes for a descriptor, in the reference's layouts."""
    pi, po = in_pack(d.format), out_pack(d.format)
    oh = out_size(d.ih, d.fh, d.dilate_h, d.stride_h, d.pad_h)
    ow = out_size(d.iw, d.fw, d.dilate_w, d.stride_w, d.pad_w)
    icpg, ocpg, g = d.ic // d.group, d.oc // d.group, d.group
    dw4 = d.format in (FMT_NCHW4, FMT_NCHW44) and g > 1 and icpg == 1 and ocpg == 1
    if d.format == FMT_NCHW:
        src = (d.n, d.ic, d.ih, d.iw)
        flt = (d.oc, d.ic, d.fh, d.fw) if g == 1 else (g, ocpg, icpg, d.fh, d.fw)
        dst = (d.n, d.oc, oh, ow)
        bias = (1, d.oc, 1, 1)
    else:
        src = (d.n, d.ic // pi, d.ih, d.iw, pi)
        dst = (d.n, d.oc // po, oh, ow, po) if po > 1 else (d.n, d.oc, oh, ow)
        bias = (1, d.oc // po, 1, 1, po) if po > 1 else (1, d.oc, 1, 1)
        if dw4:
            flt = (g // 4, 1, 1, d.fh, d.fw, 4)
        elif d.format == FMT_NCHW44:
            flt = (d.oc // 4, d.ic // 4, d.fh, d.fw, 4, 4) if g == 1 else \
                (g, ocpg // 4, icpg // 4, d.fh, d.fw, 4, 4)
        else:
            flt = (d.oc, d.ic // pi, d.fh, d.fw, pi) if g == 1 else (g, ocpg, icpg // pi, d.fh, d.fw, pi)
    if d.bias_mode == BIAS_FULL:
        bias = dst
    return src, flt, bias, dst
