"""Validates the oracle's restatement against the helper functions of the NeutronBench sources
themselves, compiled by oracle/build_ref.sh into oracle/_ref/libnts_ref.so (skipped where that
library has not been built).  CPU only."""
import ctypes
import os

import numpy as np
import pytest

import oracle

_REF = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libnts_ref.so")
pytestmark = pytest.mark.skipif(not os.path.exists(_REF), reason="oracle/_ref/libnts_ref.so not built")

_f32p = ctypes.POINTER(ctypes.c_float)
_u32p = ctypes.POINTER(ctypes.c_uint32)


@pytest.fixture(scope="module")
def ref():
    lib = ctypes.CDLL(_REF)
    lib.ref_nts_norm_degree.restype = ctypes.c_float
    lib.ref_dot_product.restype = ctypes.c_float
    return lib


def test_norm_degree_bit_exact(ref):
    n = 300
    outd = np.arange(1, n + 1, dtype=np.uint32)
    ind = (np.arange(1, n + 1, dtype=np.uint32) * 7919) % 100003 + 1
    for s in range(n):
        for d in range(0, n, 7):
            got = np.float32(ref.ref_nts_norm_degree(outd.ctypes.data_as(_u32p), ind.ctypes.data_as(_u32p), s, d))
            assert got.tobytes() == oracle.norm_degree(outd[s], ind[d]).tobytes(), (s, d)


@pytest.mark.parametrize("n", [1, 7, 8, 9, 16, 41, 128, 602])
def test_nts_comp_matches_one_documented_variant(ref, n):
    """The reference's nts_comp (AVX multiply + add, scalar tail) compiled with its own flags equals
    the oracle's fused variant bit for bit (GCC contracts the two intrinsics into an FMA), and its
    non-AVX loop likewise; the oracle's two-rounding variant differs only by that contraction."""
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    acc = rng.standard_normal(n).astype(np.float32)
    w = np.float32(rng.random())
    out = acc.copy()
    ref.ref_nts_comp(out.ctypes.data_as(_f32p), x.ctypes.data_as(_f32p), ctypes.c_float(float(w)), n)
    fused = oracle.comp(acc, x, w, fused=True)
    plain = oracle.comp(acc, x, w, fused=False)
    assert np.array_equal(out, fused) or np.array_equal(out, plain)
    assert np.allclose(out, plain, rtol=1e-6, atol=1e-7)
    out2 = acc.copy()
    ref.ref_nts_comp_non_avx256(out2.ctypes.data_as(_f32p), x.ctypes.data_as(_f32p), ctypes.c_float(float(w)), n)
    assert np.array_equal(out2, fused) or np.array_equal(out2, plain)


def test_row_aggregation_through_reference_nts_comp(ref):
    """One destination row aggregated edge by edge with the reference's nts_comp equals the
    oracle's spmm row (the order and the per-edge update are what the operators add on top)."""
    rng = np.random.default_rng(3)
    F, deg, Vs = 37, 50, 80
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    idx = rng.integers(0, Vs, deg).astype(np.uint32)
    w = rng.random(deg).astype(np.float32)
    row = np.zeros(F, dtype=np.float32)
    for e in range(deg):
        src = np.ascontiguousarray(x[idx[e]])
        ref.ref_nts_comp(row.ctypes.data_as(_f32p), src.ctypes.data_as(_f32p), ctypes.c_float(float(w[e])), F)
    off = np.array([0, deg], dtype=np.uint32)
    fused = oracle.spmm(x, w, off, idx, 1, fused=True)[0]
    plain = oracle.spmm(x, w, off, idx, 1, fused=False)[0]
    assert np.array_equal(row, fused) or np.array_equal(row, plain)


def test_nts_copy_and_dot_product(ref):
    rng = np.random.default_rng(4)
    F = 13
    table = rng.standard_normal((20, F)).astype(np.float32)
    out = np.zeros((5, F), dtype=np.float32)
    for i, s in enumerate([3, 19, 0, 7, 7]):
        ref.ref_nts_copy(out.ctypes.data_as(_f32p), ctypes.c_long(i), table.ctypes.data_as(_f32p), ctypes.c_uint32(s), F, 1)
    assert np.array_equal(out, oracle.get_feature(table, np.array([3, 19, 0, 7, 7], dtype=np.uint32)))
    a, b = table[0].copy(), table[1].copy()
    got = np.float32(ref.ref_dot_product(a.ctypes.data_as(_f32p), b.ctypes.data_as(_f32p), F))
    assert abs(float(got) - float(a.astype(np.float64) @ b.astype(np.float64))) < 1e-5
