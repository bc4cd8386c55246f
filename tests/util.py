"""Shared helpers of the test-suite: seeded random graph blocks and the error metric."""
import numpy as np


def random_block(Vd, Vs, mean_deg, seed, hub=0, dup=False, empty_frac=0.1):
    """Random bipartite CSC block: returns (co [Vd+1] uint32, ri [E] uint32 local source ids).
    `hub` > 0 gives destination 0 (if any) that many in-edges.  Some destinations are empty."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(mean_deg, Vd).astype(np.int64)
    deg[rng.random(Vd) < empty_frac] = 0
    if hub and Vd:
        deg[0] = hub
    if not dup:
        deg = np.minimum(deg, Vs)
    co = np.zeros(Vd + 1, dtype=np.int64)
    co[1:] = np.cumsum(deg)
    parts = []
    for d in range(Vd):
        if deg[d] == 0:
            continue
        if dup:
            parts.append(rng.integers(0, Vs, deg[d]))
        else:
            parts.append(rng.choice(Vs, deg[d], replace=False))
    ri = np.concatenate(parts) if parts else np.zeros(0, dtype=np.int64)
    return co.astype(np.uint32), ri.astype(np.uint32)


def planless_piece_edges(E):
    """Rows of a plan-less aggregation call (nts_spmm_gather, nts_spmm_gather_heads) with at most
    this many edges are summed as one sequential chain, in edge order; longer rows are summed in
    pieces.  None = no row is cut (calls below 65,536 edges)."""
    return 256 if E >= 1 << 16 else None


def brute_csr(co, ri, Vs):
    """Transposed structure by a stable sort of (source, edge id): (ro, ci, perm)."""
    Vd = co.size - 1
    dst_of = np.repeat(np.arange(Vd, dtype=np.int64), np.diff(co.astype(np.int64)))
    perm = np.argsort(ri.astype(np.int64), kind="stable")
    ro = np.zeros(Vs + 1, dtype=np.int64)
    ro[1:] = np.cumsum(np.bincount(ri.astype(np.int64), minlength=Vs))
    return ro.astype(np.uint32), dst_of[perm].astype(np.uint32), perm.astype(np.uint32)


def rel_err(a, b, scale=None, floor=1e-2):
    """max |a-b| / max(|a|, |b|, floor*scale): relative error that does not blow up where a sum
    cancels to (almost) zero; `scale` is the sum of the magnitudes of the terms that were added
    (default: the largest |value| of the row).  With the 1e-4 tolerance this is the bound
    |a-b| <= 1e-4 * max(|a|, |b|) + 1e-6 * sum|terms|: two fp32 summation orders of n terms differ
    by up to ~sqrt(n) ulp of the term scale."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if a.size == 0:
        return 0.0
    if scale is None:
        m = np.maximum(np.abs(a), np.abs(b))
        scale = m.max(axis=-1, keepdims=True) if a.ndim > 1 else m.max()
    den = np.maximum(np.maximum(np.abs(a), np.abs(b)), floor * np.asarray(scale, dtype=np.float64))
    den = np.maximum(den, 1e-30)
    return float((np.abs(a - b) / den).max())


def abs_term_scale(x, w, offsets, indices, rows):
    """sum_e |w[e]| * |x[indices[e], :]| per output row, in fp64: the natural error scale of a row."""
    x = np.abs(np.asarray(x, dtype=np.float64))
    out = np.zeros((rows, x.shape[1]))
    for r in range(rows):
        for e in range(int(offsets[r]), int(offsets[r + 1])):
            out[r] += (abs(float(w[e])) if w is not None else 1.0) * x[int(indices[e])]
    return out


def check(a, b, scale=None, floor=1e-2, tol=1e-4):
    """Asserts rel_err(a, b) <= tol with a short failure message (not the arrays)."""
    err = rel_err(a, b, scale, floor)
    assert err <= tol, f"max relative error {err:.3e} exceeds {tol:.0e}"
