"""Shared helpers for the parity tests: the package's portable seeded tensors, and layout converters."""
import numpy as np

from megengine_amd.synth import make_tensors, splitmix64, uniform_int  # noqa: F401


# ---- layout converters written from the closed-form definition (numpy reshape/transpose) ----

def nchw_to_packed(x, p):
    n, c, h, w = x.shape
    assert c % p == 0
    return np.ascontiguousarray(x.reshape(n, c // p, p, h, w).transpose(0, 1, 3, 4, 2))


def packed_to_nchw(x):
    n, cb, h, w, p = x.shape
    return np.ascontiguousarray(x.transpose(0, 1, 4, 2, 3).reshape(n, cb * p, h, w))


def filter_nchw_to_packed(f, p):
    """(OC, IC, FH, FW) -> (OC, IC/p, FH, FW, p); group (G, OCpg, ICpg, FH, FW) likewise."""
    if f.ndim == 4:
        oc, ic, fh, fw = f.shape
        return np.ascontiguousarray(f.reshape(oc, ic // p, p, fh, fw).transpose(0, 1, 3, 4, 2))
    g, oc, ic, fh, fw = f.shape
    return np.ascontiguousarray(f.reshape(g, oc, ic // p, p, fh, fw).transpose(0, 1, 2, 4, 5, 3))


def filter_nchw_to_nchw44(f):
    """(OC, IC, FH, FW) -> (OC/4, IC/4, FH, FW, 4ic, 4oc); group adds a leading G."""
    if f.ndim == 4:
        oc, ic, fh, fw = f.shape
        return np.ascontiguousarray(f.reshape(oc // 4, 4, ic // 4, 4, fh, fw).transpose(0, 2, 4, 5, 3, 1))
    g, oc, ic, fh, fw = f.shape
    return np.ascontiguousarray(f.reshape(g, oc // 4, 4, ic // 4, 4, fh, fw).transpose(0, 1, 3, 5, 6, 4, 2))


def filter_dw_nchw_to_dw4(f):
    """depthwise (C, 1, 1, FH, FW) -> (C/4, 1, 1, FH, FW, 4)."""
    c, _, _, fh, fw = f.shape
    return np.ascontiguousarray(f.reshape(c // 4, 4, fh, fw).transpose(0, 2, 3, 1).reshape(c // 4, 1, 1, fh, fw, 4))


def bias_to_packed(b, p):
    return np.ascontiguousarray(b.reshape(1, -1, p, 1, 1).transpose(0, 1, 3, 4, 2))
