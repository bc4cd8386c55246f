"""Seeded synthetic inputs shaped like the benchmark datasets (no dataset downloads).

Graphs come from a counter-based integer hash (splitmix64 finaliser over seed, level and edge
number), evaluated with torch int64 tensor arithmetic, so the same seed yields the same edge list
on the CPU and on the GPU.  R-MAT edges (a, b, c, d quadrant probabilities) are folded to V
vertices and relabelled by a seeded permutation so that hub vertices are not clustered at low ids.
"""
import math

import torch

_M64 = (1 << 64) - 1


def _s64(c):
    c &= _M64
    return c - (1 << 64) if c >= (1 << 63) else c


_GOLDEN = _s64(0x9E3779B97F4A7C15)
_MIX1 = _s64(0xBF58476D1CE4E5B9)
_MIX2 = _s64(0x94D049BB133111EB)


def _lshr(x, k):
    """Logical right shift of an int64 tensor."""
    return (x >> k) & ((1 << (64 - k)) - 1)


def hash64(counter, stream):
    """splitmix64 finaliser of (counter + stream * golden); int64 tensors with wrapping arithmetic."""
    z = counter + _s64(stream * 0x9E3779B97F4A7C15)
    z = z * 1 + _GOLDEN
    z = (z ^ _lshr(z, 30)) * _MIX1
    z = (z ^ _lshr(z, 27)) * _MIX2
    return z ^ _lshr(z, 31)


def uniform24(counter, stream):
    """24-bit uniform integers in [0, 2^24)."""
    return _lshr(hash64(counter, stream), 40)


def permutation(n, seed, device="cpu"):
    """Seeded permutation of range(n): argsort of hashed keys."""
    keys = hash64(torch.arange(n, dtype=torch.int64, device=device), seed * 1000003 + 17)
    return torch.argsort(keys, stable=True)


def rmat_edges(V, E, a=0.57, b=0.19, c=0.19, seed=1, device="cpu", permute=True, sort=False, distinct=False):
    """R-MAT directed edge list (src, dst) as int64 tensors of length E.  sort=True returns the list
    in (source, destination) order, the order of an edge file exported from sorted adjacency lists.
    Duplicates are kept unless distinct=True: then the list holds the first E distinct (src, dst)
    pairs of the same draw sequence (a simple graph, as the social-network datasets are), in draw
    order or, with sort=True, in (source, destination) order."""
    if distinct:
        return _rmat_distinct(V, E, a, b, c, seed, device, permute, sort)
    return _rmat_draws(V, 0, E, a, b, c, seed, device, permute, sort)


def _rmat_distinct(V, E, a, b, c, seed, device, permute, sort):
    if E > V * V:
        raise ValueError("more distinct edges asked for than vertex pairs exist")
    draws = E + E // 2 + 16
    while True:
        src, dst = _rmat_draws(V, 0, draws, a, b, c, seed, device, permute, False)
        key = src * V + dst
        del src, dst
        skey, order = torch.sort(key, stable=True)  # equal pairs stay in draw order: the first is the earliest draw
        del key
        first = torch.ones(draws, dtype=torch.bool, device=device)
        first[1:] = skey[1:] != skey[:-1]
        n_distinct = int(first.sum())
        if n_distinct >= E:
            break
        del skey, order, first
        draws = draws + draws // 3  # the same draw sequence, longer
    skey, drawn_at = skey[first], order[first]
    del order, first
    if n_distinct > E:  # keep the E pairs that were drawn first
        limit = torch.sort(drawn_at).values[E - 1]
        keep = drawn_at <= limit
        skey, drawn_at = skey[keep], drawn_at[keep]
    if not sort:
        skey = skey[torch.sort(drawn_at).indices]
    return skey // V, skey % V


def _rmat_draws(V, first, count, a, b, c, seed, device, permute, sort):
    """Draws first .. first + count - 1 of the seeded R-MAT sequence."""
    E = count
    scale = max(1, math.ceil(math.log2(V)))
    ta = int(a * (1 << 24))
    tb = int((a + b) * (1 << 24))
    tc = int((a + b + c) * (1 << 24))
    idx = torch.arange(first, first + E, dtype=torch.int64, device=device)
    src = torch.zeros(E, dtype=torch.int64, device=device)
    dst = torch.zeros(E, dtype=torch.int64, device=device)
    for level in range(scale):
        r = uniform24(idx, seed * 131 + level)
        src_bit = (r >= tb).to(torch.int64)                       # quadrants c, d
        dst_bit = (((r >= ta) & (r < tb)) | (r >= tc)).to(torch.int64)  # quadrants b, d
        src = src * 2 + src_bit
        dst = dst * 2 + dst_bit
        del r, src_bit, dst_bit
    src %= V
    dst %= V
    if permute:
        p = permutation(V, seed, device)
        src = p[src]
        dst = p[dst]
    if sort:
        order = torch.sort(src * V + dst).indices
        src, dst = src[order], dst[order]
    return src, dst


def powerlaw_symmetric_edges(V, pairs, gamma=2.5, seed=1):
    """Chung-Lu style symmetric graph: `pairs` distinct undirected pairs without self loops, returned
    as 2*pairs directed edges (both directions).  CPU, small graphs."""
    g = torch.Generator().manual_seed(seed)
    ranks = torch.arange(1, V + 1, dtype=torch.float64)
    wts = ranks.pow(-1.0 / (gamma - 1.0))
    chosen = set()
    out = []
    while len(out) < pairs:
        need = (pairs - len(out)) * 2 + 16
        u = torch.multinomial(wts, need, replacement=True, generator=g).tolist()
        v = torch.multinomial(wts, need, replacement=True, generator=g).tolist()
        for x, y in zip(u, v):
            if x == y:
                continue
            key = (x, y) if x < y else (y, x)
            if key in chosen:
                continue
            chosen.add(key)
            out.append(key)
            if len(out) == pairs:
                break
    p = permutation(V, seed).tolist()
    src = [p[x] for x, _ in out] + [p[y] for _, y in out]
    dst = [p[y] for _, y in out] + [p[x] for x, _ in out]
    return torch.tensor(src, dtype=torch.int64), torch.tensor(dst, dtype=torch.int64)


def normal_features(n, F, seed, device="cpu"):
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn(n, F, generator=g, device=device, dtype=torch.float32)


def binary_features(n, F, p, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(n, F, generator=g) < p).to(torch.float32)


def uniform_labels(n, classes, seed, device="cpu"):
    return (uniform24(torch.arange(n, dtype=torch.int64, device=device), seed * 7919 + 3) % classes).to(torch.int64)


def sample_neighbors(co, ri, dst, fanout, seed):
    """Harness-side neighbour choice for one hop (the reference's choice depends on its RNG and
    container iteration order, so the chosen lists are an input to both the oracle and the GPU path).
    co / ri: whole-graph CSC (int64 CPU tensors), dst: global ids of this hop's destinations.
    Returns (column_offset, row_indices holding GLOBAL source ids)."""
    g = torch.Generator().manual_seed(seed)
    co_l = co.tolist()
    offs = [0]
    picks = []
    for d in dst.tolist():
        lo, hi = co_l[d], co_l[d + 1]
        deg = hi - lo
        if fanout < 0 or deg <= fanout:
            picks.append(ri[lo:hi])
            offs.append(offs[-1] + deg)
        else:
            sel = torch.randperm(deg, generator=g)[:fanout]
            picks.append(ri[lo + sel])
            offs.append(offs[-1] + fanout)
    rows = torch.cat(picks) if picks else torch.zeros(0, dtype=torch.int64)
    return torch.tensor(offs, dtype=torch.int64), rows


def build_csc(src, dst, V):
    """Whole-graph CSC (column_offset [V+1], row_indices [E] = global source ids, both int64) with
    the edge order of the reference's layout: sources ascending inside a destination."""
    order = torch.sort(src, stable=True).indices
    s2, d2 = src[order], dst[order]
    perm = torch.sort(d2, stable=True).indices
    co = torch.zeros(V + 1, dtype=torch.int64, device=src.device)
    co[1:] = torch.cumsum(torch.bincount(d2, minlength=V), 0)
    return co, s2[perm]


def sample_hop(co, ri, dst, fanout, seed):
    """Vectorised neighbour choice for one hop: every destination takes all its in-neighbours when
    it has at most `fanout` of them (or fanout < 0), otherwise `fanout` distinct consecutive CSC
    positions starting at a seeded random offset (with wrap-around).  Which neighbours are chosen is
    an input to both the oracle and the GPU path, not a parity target.
    Returns (column_offset [n+1], row_indices with GLOBAL source ids), int64 on co's device."""
    deg = co[dst + 1] - co[dst]
    take = deg if fanout < 0 else torch.clamp(deg, max=fanout)
    off = torch.zeros(dst.numel() + 1, dtype=torch.int64, device=co.device)
    off[1:] = torch.cumsum(take, 0)
    E = int(off[-1])
    owner = torch.repeat_interleave(torch.arange(dst.numel(), device=co.device), take)
    j = torch.arange(E, device=co.device) - off[owner]
    start = uniform24(dst, seed * 977 + 5) % torch.clamp(deg, min=1)
    start = torch.where(deg > take, start, torch.zeros_like(start))
    pos = (start[owner] + j) % torch.clamp(deg[owner], min=1)
    return off, ri[co[dst][owner] + pos]
