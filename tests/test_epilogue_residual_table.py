"""The residual table form of the requantisation: whenever the library claims that
floor(clamp(fma(float(sfb), c, table[z]))) equals the contract with a residual, the claim is checked here against the
CPU checker for EVERY residual value on contiguous integers through every output step and on the int32 extremes; a
table with one entry moved must fail that check (the check is not vacuous); scale triples whose steps crowd together
(scale_bias / scale_dst small) must be refused rather than approximated.  Host code only: no GPU needed."""
import ctypes as C

import numpy as np
import pytest

from megengine_amd import _abi, lib
from tests.test_epilogue_linear import eval_linear


def residual_table(s_b, s_z, s_d, nl):
    c = C.c_float()
    tab = (C.c_float * 256)()
    r = lib.lib().mi355_epilogue_residual_table(s_b, s_z, s_d, nl, C.byref(c), tab)
    assert r in (0, 1), r
    return r == 1, np.float32(c.value), np.array(tab, dtype=np.float32)


def points_through_every_step(s_b, s_z, s_d, z):
    """integers around every output step of the contract for residual z (the steps sit near
    ((k - 0.5) s_d - z s_z) / s_b), and the extremes"""
    ks = np.arange(-128, 129, dtype=np.float64) - 0.5
    centers = np.round((ks * s_d - z * s_z) / s_b)
    centers = np.clip(centers, -2.0 ** 31 + 200, 2.0 ** 31 - 200).astype(np.int64)
    win = np.arange(-48, 49, dtype=np.int64)
    ext = np.array([-2 ** 31, -2 ** 31 + 1, -2 ** 30, -2 ** 24 - 1, 2 ** 24 + 1, 2 ** 30, 2 ** 31 - 1], dtype=np.int64)
    return np.unique(np.concatenate([(centers[:, None] + win[None, :]).ravel(), ext])).astype(np.int32)


def mismatches(oracle, s_b, s_z, s_d, nl, c, tab, zs):
    bad = 0
    for u in zs:
        z = int(np.int8(np.uint8(u)))
        x = points_through_every_step(s_b, s_z, s_d, z)
        want = oracle.requant(x, s_b, s_d, nl, z=np.full(x.shape, z, dtype=np.int8), scale_z=s_z)
        got = eval_linear(x, c, tab[u], nl == _abi.NL_RELU)
        bad += int(np.count_nonzero(got != want))
    return bad


def random_triples(n, seed):
    """scale_bias / scale_dst log-uniform in [5e-3, 0.5], scale_z and scale_dst log-uniform in [1e-3, 5e-2]"""
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(n):
        c0 = np.exp(rng.uniform(np.log(5e-3), np.log(0.5)))
        s_d = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        s_z = float(np.float32(np.exp(rng.uniform(np.log(1e-3), np.log(5e-2)))))
        out.append((float(np.float32(c0 * s_d)), s_z, s_d))
    return out


# scale_bias, scale_z, scale_dst: round decimal ratios put steps exactly on integers, where the literal chain's
# roundings decide each one -- such triples are mostly refused
FIXED = [(2e-4, 0.02, 0.01), (0.5, 0.25, 1.0), (1e-3, 0.05, 0.02), (2.8e-4, 1.8e-3, 1.27e-2), (2e-4, 0.013, 0.0071),
         (3.2e-6, 6.6e-3, 1.1e-2)]
PROVED = (2e-4, 0.013, 0.0071)


def test_claimed_tables_equal_the_contract(oracle):
    found = total = 0
    for i, (s_b, s_z, s_d) in enumerate(FIXED + random_triples(16, 11)):
        for nl in (_abi.NL_IDENTITY, _abi.NL_RELU):
            ok, c, tab = residual_table(s_b, s_z, s_d, nl)
            if i >= len(FIXED):
                total += 1
                found += ok
            if not ok:
                continue
            assert c > 0
            # every residual value for the first triples, every eighth (and the ends) for the rest
            zs = range(256) if i < 8 else sorted(set(range(0, 256, 8)) | {127, 128, 255})
            assert mismatches(oracle, s_b, s_z, s_d, nl, c, tab, zs) == 0, (s_b, s_z, s_d, nl)
    assert found >= 0.6 * total, (found, total)  # not vacuous on ordinary (random) scales


def test_a_wrong_entry_is_caught(oracle):
    s_b, s_z, s_d = PROVED
    ok, c, tab = residual_table(s_b, s_z, s_d, _abi.NL_RELU)
    assert ok
    for u in (0, 77, 128, 255):
        moved = tab.copy()
        moved[u] = np.float32(moved[u] + c)  # one accumulator unit: every step of this z moves by one
        assert mismatches(oracle, s_b, s_z, s_d, _abi.NL_RELU, c, moved, [u]) > 0
        assert mismatches(oracle, s_b, s_z, s_d, _abi.NL_RELU, c, tab, [u]) == 0
    # and the entries belong to their own z: neighbours differ by about s_z / s_d
    d = np.diff(tab[:128].astype(np.float64))
    assert np.allclose(d, s_z / s_d, rtol=0.05)


def test_refuses_what_it_cannot_prove():
    # many accumulator units per output step: the literal chain's own roundings move steps that an offset cannot follow
    for s_b, s_z, s_d in ((8.5e-6, 4.6e-2, 5.9e-3), (1.7e-6, 2.3e-2, 4.8e-3), (1e-9, 0.01, 1.0)):
        assert not residual_table(s_b, s_z, s_d, _abi.NL_RELU)[0]
    c = C.c_float()
    tab = (C.c_float * 256)()
    L = lib.lib()
    assert L.mi355_epilogue_residual_table(1.0, 1.0, 1.0, _abi.NL_H_SWISH, C.byref(c), tab) < 0
    assert L.mi355_epilogue_residual_table(1.0, 1.0, 1.0, _abi.NL_RELU, None, tab) < 0
    assert L.mi355_epilogue_residual_table(1.0, 1.0, 1e30, _abi.NL_RELU, C.byref(c), tab) == 0


def test_repeated_queries_agree():
    a = residual_table(*PROVED, _abi.NL_RELU)
    b = residual_table(*PROVED, _abi.NL_RELU)
    assert a[0] and b[0] and a[1] == b[1] and np.array_equal(a[2], b[2])
