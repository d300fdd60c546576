"""GPU-side helpers for the parity tests: run a descriptor through the C ABI and through the CPU
checker on the same seeded bytes and compare bit for bit."""
import sys

import numpy as np
import torch

from megengine_amd import _abi, lib, ops
from tests import util


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def to_dev(x):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).cuda()


def pad_batch(x, stride_n):
    """(n, ...) array -> (n, stride_n) array with the payload at the front of every row."""
    n = x.shape[0]
    out = np.zeros((n, stride_n), dtype=x.dtype)
    out[:, : x[0].size] = x.reshape(n, -1)
    return out


def run_gpu(desc, src, flt, bias, z, algo=None, tile=None):
    a = None
    if algo is not None:
        a, _ = ops.conv_bias_query(desc, algo)
        if tile is not None:
            a.tile_cfg = tile
    dst = ops.conv_bias_exec(desc, to_dev(src), to_dev(flt), to_dev(bias), to_dev(z), algo=a)
    torch.cuda.synchronize()
    return dst.cpu().numpy()


def check_case(oracle, desc, seed=1, algo=None, tile=None, tag="", **ranges):
    if tile is not None and not lib.tile_usable(desc, tile):
        return None  # this tile is not an algorithm for this problem: exec would refuse it (tested on its own)
    say("case", tag, "fmt", desc.format, "n", desc.n, "ic", desc.ic, "hw", desc.ih, desc.iw, "oc", desc.oc, "f",
        desc.fh, desc.fw, "g", desc.group, "s", desc.stride_h, "p", desc.pad_h, "nl", desc.nonline, "z", desc.has_z,
        "algo", algo, "tile", tile, "seed", seed)
    src, flt, bias, z = util.make_tensors(desc, seed=seed, **ranges)
    if desc.src_stride_n:
        src = pad_batch(src, desc.src_stride_n)
    if desc.has_z and desc.z_stride_n:
        z = pad_batch(z, desc.z_stride_n)
    want = oracle.conv_bias(desc, src, flt, bias, z)
    got = run_gpu(desc, src, flt, bias, z, algo=algo, tile=tile)
    if desc.dst_stride_n:
        per_n = want[0].size
        got = got[:, :per_n].reshape(want.shape)
    assert got.shape == want.shape
    if desc.dst_dtype == _abi.DT_F32:
        # the float running sum of the reference and the exact sum scaled once agree to the tolerance of the
        # reference's own checker (1e-3 relative to max(|a|, |b|, 1))
        err = np.abs(got - want) / np.maximum(np.maximum(np.abs(got), np.abs(want)), 1.0)
        assert float(err.max()) <= 1e-3, "float dst: max relative error %g" % float(err.max())
        return want
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        raise AssertionError("%d / %d mismatches, first at %s: got %d want %d" % (
            len(bad), want.size, bad[0], got[tuple(bad[0])], want[tuple(bad[0])]))
    return want
