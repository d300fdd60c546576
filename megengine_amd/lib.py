"""ctypes binding of the C-ABI shared library (libmi355_convbias.so).

The library is built in-tree by `python -m megengine_amd.build` (or __graft_entry__.build()).
Loading fails loudly when it is missing: there is no CPU or PyTorch fallback for the hot path.
"""
import ctypes as C
import os

from . import _abi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355_convbias.so")
_LIB = None

# every symbol declared in include/mi355_convbias.h
EXPORTS = [
    "mi355_abi_version", "mi355_status_string", "mi355_last_error", "mi355_get_device_info", "mi355_stream_probe",
    "mi355_convbias_deduce_out", "mi355_convbias_algo_count", "mi355_convbias_algo_name",
    "mi355_convbias_algo_usable", "mi355_convbias_s8_query", "mi355_convbias_s8_exec",
    "mi355_igemm_tile_count", "mi355_igemm_tile_name", "mi355_igemm_tile_usable", "mi355_epilogue_linear_form", "mi355_epilogue_residual_table",
    "mi355_relayout_deduce", "mi355_relayout_exec", "mi355_requant_s32_s8_exec", "mi355_requant_s8_s8_exec", "mi355_elemwise_q_exec",
    "mi355_convbias_s8_profile",
    "mi355_pooling_deduce_out", "mi355_pooling_s8_exec", "mi355_typecvt_f32_s8_exec", "mi355_typecvt_s8_f32_exec",
    "mi355_static_workspace_bytes", "mi355_convbias_s8_exec_static_workspace",
    "mi355_epilogue_quotient_form", "mi355_convbias_s8_preprocess_size", "mi355_convbias_s8_preprocess", "mi355_convbias_s8_exec_preprocessed",
]


class Mi355Error(RuntimeError):
    def __init__(self, status, msg):
        super().__init__("mi355 status %d (%s): %s" % (status, _status_str(status), msg))
        self.status = status


def _status_str(st):
    return lib().mi355_status_string(st).decode()


def lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "HIP extension %s is missing: build it with `python -m megengine_amd.build` "
            "(there is no fallback path)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    P = C.POINTER
    L.mi355_abi_version.restype = C.c_int
    L.mi355_status_string.restype = C.c_char_p
    L.mi355_status_string.argtypes = [C.c_int]
    L.mi355_last_error.restype = C.c_char_p
    L.mi355_get_device_info.argtypes = [C.c_int, P(_abi.DeviceInfo)]
    L.mi355_stream_probe.restype = C.c_int
    L.mi355_stream_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64]
    L.mi355_convbias_deduce_out.argtypes = [P(_abi.ConvDesc), P(C.c_uint32), P(C.c_uint32)]
    L.mi355_convbias_algo_count.restype = C.c_int
    L.mi355_convbias_algo_name.restype = C.c_char_p
    L.mi355_convbias_algo_name.argtypes = [C.c_int]
    L.mi355_convbias_algo_usable.argtypes = [P(_abi.ConvDesc), C.c_int]
    L.mi355_convbias_s8_query.argtypes = [P(_abi.ConvDesc), C.c_int, P(_abi.Algo), P(C.c_size_t)]
    L.mi355_convbias_s8_exec.argtypes = [C.c_void_p, P(_abi.ConvDesc), P(_abi.Algo), C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    L.mi355_static_workspace_bytes.restype = C.c_size_t
    L.mi355_convbias_s8_exec_static_workspace.argtypes = [C.c_void_p, P(_abi.ConvDesc), P(_abi.Algo), C.c_void_p, C.c_void_p,
                                                          C.c_void_p, C.c_void_p, C.c_void_p]
    L.mi355_convbias_s8_preprocess_size.argtypes = [P(_abi.ConvDesc), P(_abi.Algo), P(C.c_size_t)]
    L.mi355_convbias_s8_preprocess.argtypes = [C.c_void_p, P(_abi.ConvDesc), P(_abi.Algo), C.c_void_p, C.c_void_p, C.c_size_t]
    L.mi355_convbias_s8_exec_preprocessed.argtypes = [C.c_void_p, P(_abi.ConvDesc), P(_abi.Algo), C.c_void_p, C.c_void_p,
                                                      C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    L.mi355_convbias_s8_profile.argtypes = [C.c_void_p, P(_abi.ConvDesc), P(_abi.Algo), C.c_void_p, C.c_void_p,
                                            C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int,
                                            P(C.c_float)]
    L.mi355_igemm_tile_count.restype = C.c_int
    L.mi355_igemm_tile_name.restype = C.c_char_p
    L.mi355_igemm_tile_name.argtypes = [C.c_int]
    L.mi355_igemm_tile_usable.argtypes = [P(_abi.ConvDesc), C.c_int]
    L.mi355_epilogue_quotient_form.restype = C.c_int
    L.mi355_epilogue_quotient_form.argtypes = [C.c_float, P(C.c_float), P(C.c_float)]
    L.mi355_epilogue_residual_table.restype = C.c_int
    L.mi355_epilogue_residual_table.argtypes = [C.c_float, C.c_float, C.c_float, C.c_uint32, P(C.c_float), P(C.c_float)]
    L.mi355_epilogue_linear_form.restype = C.c_int
    L.mi355_epilogue_linear_form.argtypes = [C.c_float, C.c_float, C.c_uint32, P(C.c_float), P(C.c_float)]
    L.mi355_relayout_deduce.argtypes = [P(_abi.RelayoutDesc), P(C.c_uint32), P(C.c_uint32)]
    L.mi355_relayout_exec.argtypes = [C.c_void_p, P(_abi.RelayoutDesc), C.c_void_p, C.c_void_p]
    L.mi355_requant_s32_s8_exec.argtypes = [C.c_void_p, P(_abi.RequantDesc), C.c_void_p, C.c_void_p, C.c_void_p]
    L.mi355_requant_s8_s8_exec.argtypes = [C.c_void_p, P(_abi.RequantDesc), C.c_void_p, C.c_void_p, C.c_void_p]
    L.mi355_elemwise_q_exec.argtypes = [C.c_void_p, P(_abi.ElemwiseDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    L.mi355_pooling_deduce_out.argtypes = [P(_abi.PoolingDesc), P(C.c_uint32), P(C.c_uint32)]
    L.mi355_pooling_s8_exec.argtypes = [C.c_void_p, P(_abi.PoolingDesc), C.c_void_p, C.c_void_p]
    L.mi355_typecvt_f32_s8_exec.argtypes = [C.c_void_p, C.c_uint64, C.c_float, C.c_void_p, C.c_void_p]
    L.mi355_typecvt_s8_f32_exec.argtypes = [C.c_void_p, C.c_uint64, C.c_float, C.c_void_p, C.c_void_p]
    if L.mi355_abi_version() != _abi.ABI_VERSION:
        raise RuntimeError("ABI version mismatch: library %d, binding %d" % (L.mi355_abi_version(), _abi.ABI_VERSION))
    _LIB = L
    return L


def check(st):
    if st != 0:
        raise Mi355Error(st, lib().mi355_last_error().decode())


def algo_names():
    L = lib()
    return [L.mi355_convbias_algo_name(i).decode() for i in range(L.mi355_convbias_algo_count())]


def tile_names():
    L = lib()
    return [L.mi355_igemm_tile_name(i).decode() for i in range(L.mi355_igemm_tile_count())]


def tile_usable(desc, tile):
    """True if the MFMA algorithm runs `desc` on exactly this tile (a forced tile that cannot is MI355_ERR_ALGO at exec)"""
    return lib().mi355_igemm_tile_usable(C.byref(desc), tile) == 0


def device_info(device=0):
    info = _abi.DeviceInfo()
    check(lib().mi355_get_device_info(device, C.byref(info)))
    return info
