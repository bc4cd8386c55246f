"""Pins the CPU oracle (oracle/nts_oracle.c) before anything is compared against it.

The reference holds no golden vectors for this path, so every function is checked against what
the mathematics fixes: closed forms, brute force on small inputs, library routines (numpy dense
products, scipy.sparse, torch.softmax / autograd) and invariants, chosen so that a dropped term, a
swapped index or a transposed operand fails at least one check.  Runs on the CPU.
"""
from fractions import Fraction

import numpy as np
import pytest
import scipy.sparse as sp
import torch

import oracle
from util import brute_csr, random_block


def _nearest_f32(fr):
    """Correctly rounded float32 of an exact Fraction."""
    c = np.float32(float(fr))
    cands = [c, np.nextafter(c, np.float32(np.inf)), np.nextafter(c, np.float32(-np.inf))]
    return min(cands, key=lambda v: abs(Fraction(float(v)) - fr))


# ---------------------------------------------------------------------------------------------
# nts_norm_degree
# ---------------------------------------------------------------------------------------------
def test_norm_degree_closed_forms():
    assert oracle.norm_degree(1, 1) == np.float32(1.0)
    assert oracle.norm_degree(4, 1) == np.float32(0.5)
    assert oracle.norm_degree(1, 4) == np.float32(0.5)
    assert oracle.norm_degree(4, 9) == _nearest_f32(Fraction(1, 6))
    assert oracle.norm_degree(16, 25) == np.float32(0.05)
    for a in range(1, 40):
        for b in range(1, 40):
            assert oracle.norm_degree(a * a, b * b) == _nearest_f32(Fraction(1, a * b)), (a, b)


def test_norm_degree_rounding_chain():
    """Each root is rounded to float before the float product: equals the chain evaluated with
    numpy scalars, and differs from sqrt of the double product on at least one pair."""
    differs = 0
    for o in range(1, 65):
        for i in range(1, 65):
            a = np.float32(np.sqrt(np.float64(o)))
            b = np.float32(np.sqrt(np.float64(i)))
            want = np.float32(1.0) / (a * b)
            got = oracle.norm_degree(o, i)
            assert got.tobytes() == np.float32(want).tobytes(), (o, i)
            alt = np.float32(1.0 / np.sqrt(np.float64(o) * np.float64(i)))
            differs += int(alt != got)
            # symmetric in its two degrees, never above one, exact bound 1/sqrt(o*i) within 2 ulp
            assert got == oracle.norm_degree(i, o)
            assert abs(float(got) - 1.0 / np.sqrt(o * i)) <= 2.5 * np.spacing(np.float32(got))
    assert differs > 0


# ---------------------------------------------------------------------------------------------
# nts_comp
# ---------------------------------------------------------------------------------------------
def test_comp_two_roundings_and_fused():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(1000).astype(np.float32)
    acc = rng.standard_normal(1000).astype(np.float32)
    w = np.float32(0.37)
    got = oracle.comp(acc, x, w, fused=False)
    assert np.array_equal(got, acc + x * w)  # numpy float32: multiply rounds, add rounds
    fused = oracle.comp(acc, x, w, fused=True)
    exact = [Fraction(float(a)) + Fraction(float(b)) * Fraction(float(w)) for a, b in zip(acc, x)]
    want = np.array([_nearest_f32(e) for e in exact], dtype=np.float32)
    assert np.array_equal(fused, want)  # one rounding of the exact a + x*w
    assert np.any(fused != got)  # the two variants are distinguishable


# ---------------------------------------------------------------------------------------------
# aggregation forward / backward
# ---------------------------------------------------------------------------------------------
def _dense(co, ri, w, Vd, Vs):
    A = np.zeros((Vd, Vs), dtype=np.float64)
    for d in range(Vd):
        for e in range(int(co[d]), int(co[d + 1])):
            A[d, int(ri[e])] += float(w[e]) if w is not None else 1.0
    return A


@pytest.mark.parametrize("F", [1, 7, 8, 19, 64])
def test_spmm_forward_equals_dense_product(F):
    Vd, Vs = 120, 200
    co, ri = random_block(Vd, Vs, 6, seed=F, hub=90, dup=True)
    rng = np.random.default_rng(F)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32)
    A = _dense(co, ri, w, Vd, Vs)
    want = A @ x.astype(np.float64)
    scale = np.abs(A) @ np.abs(x.astype(np.float64)) + 1e-30
    for fused in (False, True):
        got = oracle.spmm(x, w, co, ri, Vd, fused=fused)
        assert np.max(np.abs(got - want) / scale) < 2e-6
    # the same through scipy's CSR product (A is CSR over destinations)
    S = sp.csr_matrix((w.astype(np.float64), ri.astype(np.int64), co.astype(np.int64)), shape=(Vd, Vs))
    assert np.max(np.abs(oracle.spmm(x, w, co, ri, Vd) - S @ x.astype(np.float64)) / scale) < 2e-6
    # unweighted = weights of one
    assert np.array_equal(oracle.spmm(x, None, co, ri, Vd), oracle.spmm(x, np.ones(ri.size, np.float32), co, ri, Vd))


def test_spmm_invariants():
    Vd, Vs, F = 64, 64, 5
    co, ri = random_block(Vd, Vs, 5, seed=3)
    deg = np.diff(co.astype(np.int64))
    ones = np.ones((Vs, F), dtype=np.float32)
    out = oracle.spmm(ones, None, co, ri, Vd)
    assert np.array_equal(out, np.repeat(deg[:, None], F, 1).astype(np.float32))
    # index_base shifts the ids, not the result
    rng = np.random.default_rng(1)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32)
    base = oracle.spmm(x, w, co, ri, Vd)
    assert np.array_equal(base, oracle.spmm(x, w, co, (ri + 77).astype(np.uint32), Vd, index_base=77))
    # linearity in the input (to rounding)
    y = rng.standard_normal((Vs, F)).astype(np.float32)
    lhs = oracle.spmm((x + y).astype(np.float32), w, co, ri, Vd)
    assert np.allclose(lhs, base + oracle.spmm(y, w, co, ri, Vd), rtol=1e-5, atol=1e-5)
    # thread count does not change a bit (rows are independent)
    assert np.array_equal(base, oracle.spmm(x, w, co, ri, Vd, threads=3))
    # edge order inside a row only moves the result by rounding
    co2, ri2, w2 = co.copy(), ri.copy(), w.copy()
    for d in range(Vd):
        s, e = int(co[d]), int(co[d + 1])
        ri2[s:e] = ri[s:e][::-1]
        w2[s:e] = w[s:e][::-1]
    assert np.allclose(base, oracle.spmm(x, w2, co2, ri2, Vd), rtol=1e-5, atol=1e-6)
    # GCN weights on a k-regular ring: every output row is the mean of its k neighbours
    k = 4
    cok = (np.arange(Vd + 1) * k).astype(np.uint32)
    rik = np.concatenate([[(d + j) % Vs for j in range(k)] for d in range(Vd)]).astype(np.uint32)
    wk = np.full(rik.size, oracle.norm_degree(k, k), dtype=np.float32)
    mean = np.stack([x[(np.arange(Vd) + j) % Vs] for j in range(k)]).astype(np.float64).mean(0)
    assert np.allclose(oracle.spmm(x, wk, cok, rik, Vd), mean, rtol=1e-6, atol=1e-6)


def test_spmm_backward_is_the_adjoint():
    Vd, Vs, F = 90, 140, 6
    co, ri = random_block(Vd, Vs, 5, seed=8, hub=70, dup=True)
    ro, ci, perm = brute_csr(co, ri, Vs)
    rng = np.random.default_rng(2)
    ewf = rng.random(ri.size).astype(np.float32)
    ewb = ewf[perm]
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    g = rng.standard_normal((Vd, F)).astype(np.float32)
    y = oracle.spmm(x, ewf, co, ri, Vd)
    gin = oracle.spmm(g, ewb, ro, ci, Vs)
    A = _dense(co, ri, ewf, Vd, Vs)
    want = A.T @ g.astype(np.float64)
    assert np.allclose(gin, want, rtol=1e-5, atol=1e-5)
    lhs = (y.astype(np.float64) * g).sum()
    rhs = (x.astype(np.float64) * gin).sum()
    assert abs(lhs - rhs) < 1e-4 * max(abs(lhs), 1.0)
    # push-mode formula (scatter with the forward weights) equals pull mode
    assert np.allclose(oracle.spmm_push(g, ewf, co, ri, Vs), gin, rtol=1e-5, atol=1e-5)
    # finite differences of L = sum(y * g) with respect to x
    eps = 1e-2
    for (r, c) in [(0, 0), (17, 3), (139, 5)]:
        xp = x.copy()
        xp[r, c] += eps
        lp = (oracle.spmm(xp, ewf, co, ri, Vd).astype(np.float64) * g).sum()
        assert abs((lp - lhs) / eps - gin[r, c]) < 5e-3 * max(1.0, abs(gin[r, c]))


# ---------------------------------------------------------------------------------------------
# full-graph chunk layout
# ---------------------------------------------------------------------------------------------
def test_build_chunk_brute_force():
    V = 50
    rng = np.random.default_rng(4)
    E = 400
    src = np.sort(rng.integers(0, V, E)).astype(np.uint32)  # COO order: ascending source
    dst = rng.integers(0, V, E).astype(np.uint32)
    outd, ind = oracle.degrees(src, dst, V)
    assert np.array_equal(outd, np.maximum(np.bincount(src, minlength=V), 1))
    assert np.array_equal(ind, np.maximum(np.bincount(dst, minlength=V), 1))
    ch = oracle.build_chunk(src, dst, V, outd, ind)
    # CSC rows: edges of that destination in COO order; CSR rows likewise
    for v in range(V):
        es = [j for j in range(E) if dst[j] == v]
        assert list(ch["ri"][ch["co"][v]:ch["co"][v + 1]]) == [int(src[j]) for j in es]
        for k, j in enumerate(es):
            assert ch["ewf"][ch["co"][v] + k] == oracle.norm_degree(outd[src[j]], ind[v])
        es = [j for j in range(E) if src[j] == v]
        assert list(ch["ci"][ch["ro"][v]:ch["ro"][v + 1]]) == [int(dst[j]) for j in es]
        for k, j in enumerate(es):
            assert ch["ewb"][ch["ro"][v] + k] == oracle.norm_degree(outd[v], ind[dst[j]])
    assert ch["co"][V] == E and ch["ro"][V] == E
    # an asymmetric pair pins which degree array belongs to which end
    s2 = np.array([0, 0, 0, 0, 1], dtype=np.uint32)
    d2 = np.array([1, 2, 3, 4, 4], dtype=np.uint32)
    o2, i2 = oracle.degrees(s2, d2, 5)
    c2 = oracle.build_chunk(s2, d2, 5, o2, i2)
    # edge 0->1: out_degree(0) = 4, in_degree(1) = 1  ->  1/2
    assert c2["ewf"][c2["co"][1]] == np.float32(0.5)
    # edges into 4 come from 0 (out 4) and 1 (out 1); in_degree(4) = 2
    assert list(c2["ewf"][c2["co"][4]:c2["co"][5]]) == [oracle.norm_degree(4, 2), oracle.norm_degree(1, 2)]


# ---------------------------------------------------------------------------------------------
# sampled-layer construction
# ---------------------------------------------------------------------------------------------
def test_postprocess_brute_force():
    rng = np.random.default_rng(5)
    V = 1000
    glob = rng.integers(0, V, 700).astype(np.uint32)
    glob[:3] = [0, 63, 64]  # word boundaries of the bitmap scan
    glob[3] = V - 1
    local, source, n = oracle.postprocess(glob, V)
    want_src = sorted(set(int(g) for g in glob))
    assert list(source) == want_src and n == len(want_src)
    assert [want_src.index(int(g)) for g in glob] == list(local)
    # empty edge list
    l0, s0, n0 = oracle.postprocess(np.zeros(0, np.uint32), V)
    assert n0 == 0 and l0.size == 0 and s0.size == 0


def test_csr_from_csc_brute_force():
    for seed, dup in ((1, False), (2, True)):
        Vd, Vs = 80, 60
        co, ri = random_block(Vd, Vs, 5, seed=seed, hub=50, dup=dup)
        ro, ci = oracle.csr_from_csc(co, ri, Vs)
        bro, bci, perm = brute_csr(co, ri, Vs)
        assert np.array_equal(ro, bro) and np.array_equal(ci, bci)
        assert ro[Vs] == ri.size == co[Vd]
        # the reference's own check (sampCSC::debug_generate_csr_from_csc): both formats hold the
        # same sorted (src, dst) multiset
        csc_pairs = sorted((int(ri[e]), d) for d in range(Vd) for e in range(int(co[d]), int(co[d + 1])))
        csr_pairs = sorted((s, int(ci[e])) for s in range(Vs) for e in range(int(ro[s]), int(ro[s + 1])))
        assert csc_pairs == csr_pairs
        # destinations ascend inside every source row
        for s in range(Vs):
            seg = ci[ro[s]:ro[s + 1]]
            assert np.all(np.diff(seg.astype(np.int64)) >= 0)
    ro, ci = oracle.csr_from_csc(np.zeros(4, np.uint32), np.zeros(0, np.uint32), 5)
    assert np.array_equal(ro, np.zeros(6, np.uint32)) and ci.size == 0


def test_layer_weights_brute_force():
    Vd, Vs, V = 40, 70, 500
    co, ri = random_block(Vd, Vs, 4, seed=9, hub=30)
    ro, ci, perm = brute_csr(co, ri, Vs)
    rng = np.random.default_rng(9)
    ids = rng.permutation(V)
    source = np.sort(ids[:Vs]).astype(np.uint32)
    destination = ids[Vs:Vs + Vd].astype(np.uint32)  # disjoint from the sources, arbitrary order
    outd = np.full(V, 12345, dtype=np.uint32)
    ind = np.full(V, 54321, dtype=np.uint32)
    ewf, ewb = oracle.layer_weights(co, ri, ro, ci, source, destination, outd, ind)
    in_cnt = np.diff(co.astype(np.int64))
    out_cnt = np.bincount(ri.astype(np.int64), minlength=Vs)
    for d in range(Vd):
        for e in range(int(co[d]), int(co[d + 1])):
            assert ewf[e] == oracle.norm_degree(out_cnt[ri[e]], in_cnt[d])
    assert np.array_equal(ewb, ewf[perm])  # identical value for the same edge in both orders
    # only the layer's own entries of the global degree arrays were overwritten
    assert np.array_equal(ind[destination], in_cnt) and np.array_equal(outd[source], out_cnt)
    untouched = np.setdiff1d(np.arange(V), np.concatenate([source, destination]))
    assert np.all(outd[untouched] == 12345) and np.all(ind[untouched] == 54321)


def test_init_co_fanout():
    gco = np.array([0, 0, 3, 10, 11, 40], dtype=np.uint32)  # degrees 0, 3, 7, 1, 29
    dst = np.array([4, 1, 0, 2, 3], dtype=np.uint32)
    assert list(oracle.init_co(gco, dst, 5)) == [0, 5, 8, 8, 13, 14]
    assert list(oracle.init_co(gco, dst, -1)) == [0, 29, 32, 32, 39, 40]
    assert list(oracle.init_co(gco, dst, 100)) == [0, 29, 32, 32, 39, 40]


# ---------------------------------------------------------------------------------------------
# batch assembly
# ---------------------------------------------------------------------------------------------
def test_feature_and_label_gather():
    rng = np.random.default_rng(6)
    feat = rng.standard_normal((300, 11)).astype(np.float32)
    ids = rng.integers(0, 300, 120).astype(np.uint32)
    assert oracle.get_feature(feat, ids).tobytes() == feat[ids].tobytes()
    lab = rng.integers(0, 40, 300).astype(np.int64)
    assert np.array_equal(oracle.get_label(lab, ids), lab[ids])
    multi = rng.integers(0, 2, (300, 5)).astype(np.int64)
    assert np.array_equal(oracle.get_label(multi, ids), multi[ids])
    assert oracle.get_feature(feat, np.zeros(0, np.uint32)).shape == (0, 11)


def test_cached_gather_equals_plain_gather():
    rng = np.random.default_rng(7)
    V, F, n_cache = 400, 9, 80
    feat = rng.standard_normal((V, F)).astype(np.float32)
    out_deg = rng.integers(0, 50, V)
    order = np.argsort(-out_deg, kind="stable").astype(np.uint32)
    hashmap = oracle.mark_cache(V, order, n_cache)
    assert np.array_equal(np.sort(hashmap[order[:n_cache]]), np.arange(n_cache))
    assert np.all(hashmap[order[n_cache:]] == 0xFFFFFFFF)
    assert out_deg[order[:n_cache]].min() >= out_deg[order[n_cache:]].max()
    cache = oracle.fill_cache(feat, order, n_cache, hashmap)
    assert np.array_equal(cache, feat[order[:n_cache]])
    src = np.sort(rng.choice(V, 150, replace=False)).astype(np.uint32)
    got, hit, miss = oracle.load_feature_cached(feat, cache, src, hashmap)
    assert got.tobytes() == feat[src].tobytes()
    both = np.concatenate([hit, miss])
    assert np.array_equal(np.sort(both), np.arange(src.size))  # every row exactly once
    assert np.all(np.diff(hit.astype(np.int64)) > 0) and np.all(np.diff(miss.astype(np.int64)) > 0)
    assert np.all(hashmap[src[hit]] != 0xFFFFFFFF) and np.all(hashmap[src[miss]] == 0xFFFFFFFF)


# ---------------------------------------------------------------------------------------------
# GAT operators
# ---------------------------------------------------------------------------------------------
def _block(seed=10, Vd=30, Vs=45):
    co, ri = random_block(Vd, Vs, 4, seed=seed, hub=25)
    dst_of = np.repeat(np.arange(Vd), np.diff(co.astype(np.int64)))
    return co, ri, dst_of, Vd, Vs


def test_scatter_and_aggregate_by_indexing():
    co, ri, dst_of, Vd, Vs = _block()
    rng = np.random.default_rng(11)
    F = 6
    xs = rng.standard_normal((Vs, F)).astype(np.float32)
    xd = rng.standard_normal((Vd, F)).astype(np.float32)
    msg = oracle.scatter_src_dst(xs, xd, co, ri)
    assert np.array_equal(msg[:, :F], xs[ri]) and np.array_equal(msg[:, F:], xd[dst_of])
    assert np.array_equal(oracle.scatter_src(xs, co, ri), xs[ri])
    mirror = rng.permutation(Vs).astype(np.uint32)
    assert np.array_equal(oracle.scatter_src(xs, co, ri, mirror), xs[mirror[ri]])
    assert np.array_equal(oracle.scatter_dst(xd, co, ri.size), xd[dst_of])
    em = rng.standard_normal((ri.size, F)).astype(np.float32)
    agg = oracle.aggregate_dst(em, co)
    want = np.zeros((Vd, F))
    np.add.at(want, dst_of, em.astype(np.float64))
    assert np.allclose(agg, want, rtol=1e-5, atol=1e-5)
    gs = oracle.gather_to_src(em, co, ri, Vs)
    want = np.zeros((Vs, F))
    np.add.at(want, ri.astype(np.int64), em.astype(np.float64))
    assert np.allclose(gs, want, rtol=1e-5, atol=1e-5)
    g2 = rng.standard_normal((ri.size, 2 * F)).astype(np.float32)
    a, b = oracle.scatter_src_dst_bwd(g2, co, ri, Vs)
    assert np.allclose(a, oracle.gather_to_src(np.ascontiguousarray(g2[:, :F]), co, ri, Vs), atol=1e-6)
    assert np.allclose(b, oracle.aggregate_dst(np.ascontiguousarray(g2[:, F:]), co), atol=1e-6)


@pytest.mark.parametrize("H", [1, 3, 4])
def test_edge_softmax_is_torch_softmax_per_segment(H):
    co, ri, dst_of, Vd, Vs = _block(seed=12 + H)
    rng = np.random.default_rng(H)
    x = (rng.standard_normal((ri.size, H)) * 4).astype(np.float32)
    x[0] += 80.0  # a large logit must not overflow
    y = oracle.edge_softmax(x, co)
    for d in range(Vd):
        s, e = int(co[d]), int(co[d + 1])
        if s == e:
            continue
        want = torch.softmax(torch.from_numpy(x[s:e]).double(), 0).numpy()
        assert np.allclose(y[s:e], want, rtol=2e-6, atol=1e-7)
        assert np.allclose(y[s:e].sum(0), 1.0, atol=1e-5)
    assert np.allclose(oracle.edge_softmax(x + np.float32(3.0), co), y, rtol=1e-4, atol=1e-6)  # shift invariance
    # single-edge segments give exactly one
    co1 = np.arange(6, dtype=np.uint32)
    assert np.array_equal(oracle.edge_softmax(x[:5], co1), np.ones((5, H), np.float32))
    # backward equals autograd of the forward
    gy = rng.standard_normal((ri.size, H)).astype(np.float32)
    gx = oracle.edge_softmax_bwd(gy, y, co)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    outs = [torch.softmax(xt[int(co[d]):int(co[d + 1])], 0) for d in range(Vd) if co[d] != co[d + 1]]
    torch.cat(outs).backward(torch.from_numpy(gy).double())
    assert np.allclose(gx, xt.grad.numpy(), rtol=1e-4, atol=1e-6)
    for d in range(Vd):  # gradients of a segment sum to zero
        s, e = int(co[d]), int(co[d + 1])
        if e > s:
            assert np.allclose(gx[s:e].sum(0), 0.0, atol=1e-5)
    assert np.array_equal(oracle.edge_softmax_bwd(gy[:5], np.ones((5, H), np.float32), co1), np.zeros((5, H), np.float32))


def test_gat_chain_matches_autograd():
    """The operator chain of the reference's GAT layer (scatter src|dst -> a-projection ->
    leaky_relu -> edge softmax -> weight the source half -> aggregate) built from the oracle's
    operators, forward and backward, equals torch autograd over the same chain written with
    index_select / index_add."""
    co, ri, dst_of, Vd, Vs = _block(seed=20)
    rng = np.random.default_rng(21)
    F = 5
    hs = rng.standard_normal((Vs, F)).astype(np.float32)
    hd = rng.standard_normal((Vd, F)).astype(np.float32)
    a = rng.standard_normal((2 * F, 1)).astype(np.float32)
    gout = rng.standard_normal((Vd, F)).astype(np.float32)
    # forward with the oracle's operators + numpy for the dense pieces
    e_msg = oracle.scatter_src_dst(hs, hd, co, ri)
    pre = e_msg @ a
    m = np.where(pre > 0, pre, np.float32(0.2) * pre).astype(np.float32)
    alpha = oracle.edge_softmax(m, co)
    e_out = (e_msg[:, :F] * alpha).astype(np.float32)
    out = oracle.aggregate_dst(e_out, co)
    # backward
    g_eout = oracle.scatter_dst(gout, co, ri.size)
    g_alpha = (g_eout * e_msg[:, :F]).sum(1, keepdims=True).astype(np.float32)
    g_m = oracle.edge_softmax_bwd(g_alpha, alpha, co)
    g_pre = (g_m * np.where(pre > 0, 1.0, 0.2)).astype(np.float32)
    g_emsg = (g_pre @ a.T).astype(np.float32)
    g_emsg[:, :F] += g_eout * alpha
    g_hs, g_hd = oracle.scatter_src_dst_bwd(g_emsg, co, ri, Vs)
    # torch autograd over the same chain
    ths = torch.from_numpy(hs).double().requires_grad_(True)
    thd = torch.from_numpy(hd).double().requires_grad_(True)
    ta = torch.from_numpy(a).double()
    src_idx = torch.from_numpy(ri.astype(np.int64))
    dst_idx = torch.from_numpy(dst_of.astype(np.int64))
    tmsg = torch.cat([ths[src_idx], thd[dst_idx]], 1)
    tm = torch.nn.functional.leaky_relu(tmsg @ ta, 0.2)
    segs = [torch.softmax(tm[int(co[d]):int(co[d + 1])], 0) for d in range(Vd) if co[d] != co[d + 1]]
    talpha = torch.cat(segs)
    tout = torch.zeros(Vd, F, dtype=torch.float64).index_add(0, dst_idx, tmsg[:, :F] * talpha)
    tout.backward(torch.from_numpy(gout).double())
    assert np.allclose(out, tout.detach().numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(g_hs, ths.grad.numpy(), rtol=1e-4, atol=1e-5)
    assert np.allclose(g_hd, thd.grad.numpy(), rtol=1e-4, atol=1e-5)
