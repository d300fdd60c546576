"""Portable seeded synthetic tensors for the workloads: the same bytes on every host, for the GPU path, the CPU parity
checker and the CPU baseline alike (splitmix64; numpy only)."""
import numpy as np

from . import _abi


def splitmix64(seed, n):
    """Portable generator: n uint64 values from splitmix64(seed) (same bytes on every host)."""
    out = np.empty(n, dtype=np.uint64)
    x = np.uint64(seed)
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        z = x + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        out = z ^ (z >> np.uint64(31))
    return out


def uniform_int(seed, shape, lo, hi, dtype):
    n = int(np.prod(shape))
    r = splitmix64(seed, n)
    v = (r % np.uint64(hi - lo + 1)).astype(np.int64) + lo
    return v.astype(dtype).reshape(shape)


def make_tensors(desc, seed=1, src_range=(-128, 127), flt_range=(-128, 127), bias_range=(-1000, 1000),
                 z_range=(-128, 127)):
    src_s, flt_s, bias_s, dst_s = _abi.conv_shapes(desc)
    src = uniform_int(seed * 4 + 0, src_s, *src_range, np.int8)
    flt = uniform_int(seed * 4 + 1, flt_s, *flt_range, np.int8)
    bias = uniform_int(seed * 4 + 2, bias_s, *bias_range, np.int32) if desc.bias_mode else None
    z = None
    if desc.has_z:
        zdt = np.int8 if desc.dst_dtype == _abi.DT_QS8 else np.int32
        z = uniform_int(seed * 4 + 3, dst_s, *z_range, zdt)
    if desc.dst_dtype == _abi.DT_F32:
        # Float32 dst: bias and z are float tensors; quarter-integer values keep them exactly representable
        bias = None if bias is None else (bias.astype(np.float32) * np.float32(0.25))
        z = None if z is None else (z.astype(np.float32) * np.float32(0.25))
    return src, flt, bias, z
