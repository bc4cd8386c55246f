"""GPU parity of the aggregation kernels (through the C ABI) against the CPU oracle.

Tolerance: max relative error <= 1e-4 in fp32 (relative to max(|a|, |b|, 1e-3 * sum of |terms|)).
Unsplit rows are additionally required to be bit-identical to the oracle's fused-multiply-add
variant: the kernel adds the edges of a row in the same order with one FMA each.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from neutronbench_amd import abi
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.layout import SpmmPlan
from util import check, abs_term_scale, brute_csr, planless_piece_edges, random_block, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _dev(a, device):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.to(device)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _run_planless(x, w, off, idx, rows, F, device, base=0, accumulate=0, out_init=None):
    dx, doff, didx = _dev(x, device), _dev(off, device), _dev(idx, device)
    dw = _dev(w, device) if w is not None else None
    out = _dev(out_init, device) if out_init is not None else torch.full((rows, F), float("nan"), device=device)
    call("nts_spmm_gather", ptr(dx), ptr(out), ptr(dw), ptr(doff), ptr(didx), base, rows, idx.size, F, accumulate,
         _stream())
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("F", [1, 2, 7, 16, 32, 41, 47, 64, 100, 128, 130, 256, 602, 1433, 2050])
@pytest.mark.parametrize("weighted", [True, False])
def test_forward_matches_oracle(device, F, weighted):
    print(f"case F={F} weighted={weighted}", flush=True)
    Vd, Vs = 300, 500
    co, ri = random_block(Vd, Vs, 12, seed=F, hub=400)
    rng = np.random.default_rng(F + 1)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32) if weighted else None
    got = _run_planless(x, w, co, ri, Vd, F, device)
    ref = oracle.spmm(x, w, co, ri, Vd)
    scale = abs_term_scale(x, w, co, ri, Vd)
    check(got, ref, scale)
    ref_fma = oracle.spmm(x, w, co, ri, Vd, fused=True)
    assert np.array_equal(got.view(np.uint32), ref_fma.view(np.uint32)), "edge order / FMA chain differs"


def test_backward_is_transposed_gather(device):
    """gin = A^T gout computed over the CSR arrays equals the oracle's pull backward, the oracle's
    push backward (to rounding) and satisfies <A x, y> = <x, A^T y>."""
    Vd, Vs, F = 257, 391, 128
    co, ri = random_block(Vd, Vs, 9, seed=5, hub=300)
    ro, ci, perm = brute_csr(co, ri, Vs)
    rng = np.random.default_rng(6)
    ewf = rng.random(ri.size).astype(np.float32)
    ewb = ewf[perm]
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    gout = rng.standard_normal((Vd, F)).astype(np.float32)
    y = _run_planless(x, ewf, co, ri, Vd, F, device)
    gin = _run_planless(gout, ewb, ro, ci, Vs, F, device)
    ref = oracle.spmm(gout, ewb, ro, ci, Vs)
    check(gin, ref, abs_term_scale(gout, ewb, ro, ci, Vs))
    push = oracle.spmm_push(gout, ewf, co, ri, Vs)
    check(gin, push, abs_term_scale(gout, ewb, ro, ci, Vs))
    lhs = float((y.astype(np.float64) * gout).sum())
    rhs = float((x.astype(np.float64) * gin).sum())
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs), 1.0)


def test_accumulate_and_index_base(device):
    Vd, Vs, F, base = 64, 90, 100, 1000
    co, ri = random_block(Vd, Vs, 7, seed=11)
    rng = np.random.default_rng(12)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32)
    init = rng.standard_normal((Vd, F)).astype(np.float32)
    got = _run_planless(x, w, co, (ri + base).astype(np.uint32), Vd, F, device, base=base, accumulate=1, out_init=init)
    ref = oracle.spmm(x, w, co, ri, Vd) + init
    check(got, ref, abs_term_scale(x, w, co, ri, Vd) + np.abs(init))
    # accumulate = 0 overwrites whatever the buffer held, including rows without edges
    got0 = _run_planless(x, w, co, (ri + base).astype(np.uint32), Vd, F, device, base=base, accumulate=0, out_init=init)
    assert np.array_equal(got0, oracle.spmm(x, w, co, ri, Vd, fused=True))


@pytest.mark.parametrize("F,chunk", [(128, 64), (602, 100), (41, 32), (16, 16), (100, 4096), (300, 48), (1000, 64),
                                     (1433, 128)])
def test_planned_split_rows(device, F, chunk):
    """Degree-bucketed schedule with hub rows split into chunks: matches the oracle, reports the
    split, and is bit-reproducible run to run (no atomics)."""
    print(f"case F={F} chunk={chunk}", flush=True)
    Vd, Vs = 500, 800
    co, ri = random_block(Vd, Vs, 20, seed=F, hub=3000, dup=True)
    rng = np.random.default_rng(F)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32)
    dx, dw, dco, dri = _dev(x, device), _dev(w, device), _dev(co, device), _dev(ri, device)
    plan = SpmmPlan(dco, Vd, ri.size, chunk)
    info = plan.info()
    deg = np.diff(co.astype(np.int64))
    assert info["split_rows"] == int((deg > chunk).sum())
    assert info["partials"] == int(np.ceil(deg[deg > chunk] / chunk).sum())
    assert info["items"] == int((deg <= chunk).sum()) + info["partials"]
    outs = []
    for _ in range(2):
        out = torch.full((Vd, F), float("nan"), device=device)
        call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, F, 0, _stream())
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    ref = oracle.spmm(x, w, co, ri, Vd)
    check(outs[0], ref, abs_term_scale(x, w, co, ri, Vd))
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    # unsplit rows keep the sequential FMA chain
    ref_fma = oracle.spmm(x, w, co, ri, Vd, fused=True)
    keep = deg <= chunk
    assert np.array_equal(outs[0][keep].view(np.uint32), ref_fma[keep].view(np.uint32))
    # accumulate adds to the existing output, split rows included
    init = rng.standard_normal((Vd, F)).astype(np.float32)
    out = _dev(init, device)
    call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, F, 1, _stream())
    torch.cuda.synchronize()
    check(out.cpu().numpy(), ref + init, abs_term_scale(x, w, co, ri, Vd) + np.abs(init))
    plan.close()


@pytest.mark.parametrize("F,hubs,piece", [(16, (60000, 20001), 256), (100, (60000, 20001), 256),
                                          (128, (60000, 20001), 256), (602, (60000, 20001), 256),
                                          (100, (3000000, 2000000), 256)])     # rows of millions of edges (pieces ordered by source)
def test_planless_call_balances_hub_rows_on_the_device(device, F, hubs, piece):
    """nts_spmm_gather without a plan: above 65,536 edges rows longer than 256 edges are cut into
    pieces on the device (partial sums + ordered second stage).  Short rows keep the sequential FMA chain bit for
    bit; long rows match within the fp32 tolerance; accumulate still adds; two runs give identical
    bits."""
    print(f"case F={F} hubs={hubs}", flush=True)
    rng = np.random.default_rng(F)
    Vd, Vs = 3000, 5000
    deg = rng.integers(0, 40, Vd)
    deg[[5, 77, 1500, 2999]] = [hubs[0], piece + 1, piece, hubs[1]]  # hubs, and both sides of the piece size
    deg[100:110] = 0
    co = np.zeros(Vd + 1, dtype=np.uint32)
    co[1:] = np.cumsum(deg)
    E = int(co[-1])
    assert planless_piece_edges(E) == piece
    ri = rng.integers(0, Vs, E).astype(np.uint32)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(E).astype(np.float32)
    got = _run_planless(x, w, co, ri, Vd, F, device)
    again = _run_planless(x, w, co, ri, Vd, F, device)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    scale = abs_term_scale(x, w, co, ri, Vd)

    def expected(weights):
        """The oracle's sequential fp32 sums; for rows of more than 100,000 edges, where such a chain
        is itself off by more than the tolerance, the exact sum rounded once."""
        want = oracle.spmm(x, weights, co, ri, Vd)
        for r in np.flatnonzero(deg > 100000):
            sl = slice(int(co[r]), int(co[r + 1]))
            rows = x[ri[sl]].astype(np.float64)
            want[r] = (rows * weights[sl, None] if weights is not None else rows).sum(0)
        return want

    check(got, expected(w), scale)
    short = deg <= piece
    ref_fma = oracle.spmm(x, w, co, ri, Vd, fused=True)
    assert np.array_equal(got[short].view(np.uint32), ref_fma[short].view(np.uint32))
    assert not got[100:110].any()
    # exact value of the hub rows in fp64: the pieced sum must not be less accurate than the chain
    for r in (5, 2999):
        sl = slice(int(co[r]), int(co[r + 1]))
        exact = (x[ri[sl]].astype(np.float64) * w[sl, None]).sum(0)
        assert np.max(np.abs(got[r] - exact) / np.maximum(np.abs(exact), 1e-2 * scale[r])) <= TOL
    init = rng.standard_normal((Vd, F)).astype(np.float32)
    acc = _run_planless(x, w, co, ri, Vd, F, device, accumulate=1, out_init=init)
    check(acc, expected(w) + init, scale + np.abs(init))
    # unweighted
    got_u = _run_planless(x, None, co, ri, Vd, F, device)
    check(got_u, expected(None), abs_term_scale(x, None, co, ri, Vd))


def test_invariants(device):
    """All-ones input with unit weights gives the degree; GCN weights on a k-regular ring average."""
    Vd = Vs = 128
    F = 64
    k = 4
    co = (np.arange(Vd + 1) * k).astype(np.uint32)
    ri = np.concatenate([[(d + j) % Vs for j in range(k)] for d in range(Vd)]).astype(np.uint32)
    ones = np.ones((Vs, F), dtype=np.float32)
    got = _run_planless(ones, None, co, ri, Vd, F, device)
    assert np.array_equal(got, np.full((Vd, F), float(k), dtype=np.float32))
    w = np.full(ri.size, oracle.norm_degree(k, k), dtype=np.float32)
    x = np.random.default_rng(1).standard_normal((Vs, F)).astype(np.float32)
    got = _run_planless(x, w, co, ri, Vd, F, device)
    mean = np.stack([x[(np.arange(Vd) + j) % Vs] for j in range(k)]).mean(0)
    check(got, mean)


def test_empty_and_error_paths(device):
    F = 8
    x = torch.zeros(4, F, device=device)
    out = torch.zeros(4, F, device=device)
    off = torch.zeros(5, dtype=torch.int32, device=device)
    idx = torch.zeros(1, dtype=torch.int32, device=device)
    s = _stream()
    # rows = 0 and E = 0 are legal no-ops / zero fills
    assert abi.status("nts_spmm_gather", ptr(x), ptr(out), 0, ptr(off), ptr(idx), 0, 0, 0, F, 0, s) == abi.NTS_OK
    out.fill_(5.0)
    assert abi.status("nts_spmm_gather", ptr(x), ptr(out), 0, ptr(off), 0, 0, 4, 0, F, 0, s) == abi.NTS_OK
    torch.cuda.synchronize()
    assert float(out.abs().sum()) == 0.0
    # F = 0 and null pointers are rejected with a status, not a crash
    assert abi.status("nts_spmm_gather", ptr(x), ptr(out), 0, ptr(off), ptr(idx), 0, 4, 0, 0, 0, s) == abi.NTS_ERR_INVALID
    assert abi.status("nts_spmm_gather", ptr(x), 0, 0, ptr(off), ptr(idx), 0, 4, 0, F, 0, s) == abi.NTS_ERR_INVALID
    assert "null" in abi.last_error() or "F" in abi.last_error()
    # plan creation rejects inconsistent offsets
    handle = ctypes.c_void_p()
    assert abi.status("nts_spmm_plan_create", ctypes.byref(handle), ptr(off), 4, 7, 0, s) == abi.NTS_ERR_INVALID


@pytest.mark.parametrize("F,chunk,slabs,sorted_rows", [(128, 64, 4, True), (602, 100, 8, True), (41, 32, 16, True),
                                                       (100, 64, 8, False), (16, 16, 3, True), (64, 48, 32, True),
                                                       (602, 64, 4, False), (128, 96, 16, False)])
def test_cache_aware_plan(device, F, chunk, slabs, sorted_rows):
    """Source-range ("slab") schedule: same results as the oracle to tolerance, bit-reproducible, also
    for rows whose indices do not ascend (cut in the schedule's own sorted copy)."""
    print(f"case F={F} chunk={chunk} slabs={slabs} sorted={sorted_rows}", flush=True)
    Vd, Vs = 400, 900
    co, ri = random_block(Vd, Vs, 25, seed=F + slabs, hub=2500, dup=True)
    if sorted_rows:
        for d in range(Vd):
            ri[co[d]:co[d + 1]] = np.sort(ri[co[d]:co[d + 1]])
    rng = np.random.default_rng(F)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32)
    dx, dw, dco, dri = _dev(x, device), _dev(w, device), _dev(co, device), _dev(ri, device)
    plan = SpmmPlan(dco, Vd, ri.size, chunk, dri, Vs, slabs)
    info = plan.info()
    deg = np.diff(co.astype(np.int64))
    # With 8 or more source ranges, rows of more than chunk/4 edges are cut as well, at a quarter as
    # many (wider) ranges, unless all their edges fall into one of those.  Rows that do not ascend
    # are cut in the schedule's own sorted copy of the indices, so they behave like sorted ones.
    second_tier = slabs >= 8
    whole_up_to = chunk // 4 if second_tier else chunk
    long_rows = int((deg > chunk).sum())
    plain = int(np.ceil(deg[deg > chunk] / chunk).sum())
    if second_tier:
        medium = int(((deg > whole_up_to) & (deg <= chunk)).sum())
        assert long_rows <= info["split_rows"] <= long_rows + medium
        assert plain <= info["partials"] <= plain + long_rows * slabs + medium * (slabs // 4)
    else:
        assert info["split_rows"] == long_rows
        assert plain <= info["partials"] <= plain + info["split_rows"] * slabs
    outs = []
    for _ in range(2):
        out = torch.full((Vd, F), float("nan"), device=device)
        call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, F, 0, _stream())
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    check(outs[0], oracle.spmm(x, w, co, ri, Vd), abs_term_scale(x, w, co, ri, Vd))
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    keep = deg <= whole_up_to
    assert np.array_equal(outs[0][keep].view(np.uint32), oracle.spmm(x, w, co, ri, Vd, fused=True)[keep].view(np.uint32))
    plan.close()


@pytest.mark.parametrize("runs,pad", [("1", "1"), ("0", "0")])
def test_forced_kernel_variants_in_a_fresh_process(device, runs, pad):
    """A schedule picks by itself whether rows are loaded once per run of equal indices and whether
    widths off 16-byte boundaries are gathered from a padded copy (both when at least 1 edge in 20
    repeats its predecessor's index).  NTS_SPMM_RUNS / NTS_SPMM_PAD (read once per process) force the
    choice: both settings pass the same parity cases, bit-exact rows included."""
    import os
    import subprocess
    import sys

    env = dict(os.environ, NTS_SPMM_RUNS=runs, NTS_SPMM_PAD=pad)
    here = os.path.dirname(os.path.abspath(__file__))
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(here, "test_gpu_aggregate.py"), "-q", "-x", "-m", "gpu",
                        "-k", "planned_split_rows or cache_aware or random_shapes or runs_of_equal", "--timeout", "120",
                        "--timeout-method", "thread"], env=env, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-1500:]


@pytest.mark.parametrize("F", [16, 100, 128, 130, 200, 301, 602, 256, 1433])
def test_runs_of_equal_indices_are_loaded_once_and_added_edge_by_edge(device, F):
    """A multigraph block with sorted rows: two thirds of the edges repeat their predecessor's index,
    so the schedule turns on the one-load-per-run kernel (and, for widths that are not multiples of
    four, the padded copy of the input).  Every edge is still added with its own weight in edge order:
    rows that are not cut equal the oracle's fused chain bit for bit."""
    print(f"case F={F}", flush=True)
    rng = np.random.default_rng(F)
    Vd, Vs, chunk, slabs = 600, 400, 64, 8
    deg = rng.integers(0, 60, Vd)
    deg[[3, 299]] = [5000, 700]
    co = np.zeros(Vd + 1, dtype=np.uint32)
    co[1:] = np.cumsum(deg)
    ri = np.concatenate([np.sort(np.repeat(rng.integers(0, Vs, (d + 2) // 3), 3)[:d]) for d in deg]).astype(np.uint32)
    assert (ri[1:] == ri[:-1]).mean() > 0.5
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32)
    dx, dw, dco, dri = _dev(x, device), _dev(w, device), _dev(co, device), _dev(ri, device)
    plan = SpmmPlan(dco, Vd, ri.size, chunk, dri, Vs, slabs)
    ref_fma = oracle.spmm(x, w, co, ri, Vd, fused=True)
    scale = abs_term_scale(x, w, co, ri, Vd)
    for accumulate in (0, 1):
        init = rng.standard_normal((Vd, F)).astype(np.float32)
        out = _dev(init, device) if accumulate else torch.full((Vd, F), float("nan"), device=device)
        call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, F, accumulate,
             _stream())
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        if accumulate:
            check(got, oracle.spmm(x, w, co, ri, Vd) + init, scale + np.abs(init))
        else:
            check(got, oracle.spmm(x, w, co, ri, Vd), scale)
            keep = deg <= chunk // 4
            assert keep.sum() > 100
            assert np.array_equal(got[keep].view(np.uint32), ref_fma[keep].view(np.uint32))
    # unweighted through the same schedule
    out = torch.full((Vd, F), float("nan"), device=device)
    call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), 0, ptr(dco), ptr(dri), 0, F, 0, _stream())
    torch.cuda.synchronize()
    check(out.cpu().numpy(), oracle.spmm(x, None, co, ri, Vd), abs_term_scale(x, None, co, ri, Vd))
    plan.close()


def test_one_plan_called_from_two_streams(device):
    """A plan's scratch (partial sums, padded input copy) is shared by all calls on it.  Calls from
    different streams are ordered by the library (the later stream waits, on the device, for the
    earlier call's last kernel), so two streams that use one plan without any host-side wait still
    get the results of calls made one at a time."""
    rng = np.random.default_rng(77)
    Vd, Vs, F, chunk, slabs = 30000, 20000, 602, 64, 8
    deg = rng.integers(0, 120, Vd)
    deg[[5, 77, 1500]] = [200000, 50000, 9000]
    co = np.zeros(Vd + 1, dtype=np.uint32)
    co[1:] = np.cumsum(deg)
    ri = np.concatenate([np.sort(rng.integers(0, Vs, d)) for d in deg]).astype(np.uint32)
    w = rng.random(ri.size).astype(np.float32)
    xs = [rng.standard_normal((Vs, F)).astype(np.float32) for _ in range(2)]
    dw, dco, dri = _dev(w, device), _dev(co, device), _dev(ri, device)
    dxs = [_dev(x, device) for x in xs]
    plan = SpmmPlan(dco, Vd, ri.size, chunk, dri, Vs, slabs)
    assert plan.info()["partials"] > 20000
    want = []
    for dx in dxs:  # one at a time
        out = torch.empty(Vd, F, device=device)
        call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, F, 0, _stream())
        torch.cuda.synchronize()
        want.append(out.cpu().numpy())
    streams = [torch.cuda.Stream(device=device) for _ in range(2)]
    outs = [torch.empty(Vd, F, device=device) for _ in range(2)]
    torch.cuda.synchronize()
    for _ in range(6):  # alternate streams back to back, no host wait in between
        for k in range(2):
            call("nts_spmm_gather_planned", plan.handle, ptr(dxs[k]), ptr(outs[k]), ptr(dw), ptr(dco), ptr(dri), 0, F, 0,
                 streams[k].cuda_stream)
    torch.cuda.synchronize()
    for k in range(2):
        assert np.array_equal(outs[k].cpu().numpy().view(np.uint32), want[k].view(np.uint32)), f"stream {k}"
    plan.close()


def test_scratch_pool_is_kept_between_calls_and_can_be_trimmed(device):
    """Calls that cut hub rows take their scratch from the library's own pool: it is kept after the
    call (the next call does not pay for a fresh allocation) and nts_scratch_trim hands it back."""
    rng = np.random.default_rng(7)
    Vd, Vs, F = 2000, 3000, 256
    deg = rng.integers(0, 30, Vd)
    deg[3] = 3_000_000  # about 11,700 pieces of 256 edges -> ~24 MB of partial sums
    co = np.zeros(Vd + 1, dtype=np.uint32)
    co[1:] = np.cumsum(deg)
    ri = rng.integers(0, Vs, int(co[-1])).astype(np.uint32)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    call("nts_scratch_trim")
    first = _run_planless(x, None, co, ri, Vd, F, device)  # synchronises before it returns
    held = torch.cuda.mem_get_info()[0]
    call("nts_scratch_trim")
    released = torch.cuda.mem_get_info()[0] - held
    assert released >= 8 << 20, released  # the pool still had the partial-sum scratch, and gave it back
    again = _run_planless(x, None, co, ri, Vd, F, device)
    assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
    call("nts_scratch_trim")


@pytest.mark.parametrize("seed", range(40))
def test_random_shapes_planned_and_planless_agree_with_the_oracle(device, seed):
    """Random block shapes, widths, piece lengths, range counts (also ones that 4 does not divide),
    sorted and unsorted rows, weighted or not, accumulating or not: the planned and the plan-less
    call both match the oracle, and rows that no schedule cuts match it bit for bit."""
    from neutronbench_amd.layout import SpmmPlan

    rng = np.random.default_rng(1000 + seed)
    Vd, Vs = int(rng.integers(1, 700)), int(rng.integers(1, 900))
    F = int(rng.choice([1, 3, 4, 8, 20, 33, 64, 100, 128, 129, 300, 602]))
    chunk = int(rng.choice([4, 16, 50, 128, 512]))
    slabs = int(rng.choice([1, 2, 3, 8, 9, 10, 12, 32, 100]))
    co, ri = random_block(Vd, Vs, float(rng.choice([0.5, 6, 40])), seed=seed, hub=int(rng.choice([0, 300, 5000])), dup=True)
    if rng.random() < 0.5:
        for d in range(Vd):
            ri[co[d]:co[d + 1]] = np.sort(ri[co[d]:co[d + 1]])
    weighted, accumulate = bool(rng.random() < 0.7), int(rng.random() < 0.5)
    print(f"case Vd={Vd} Vs={Vs} E={ri.size} F={F} chunk={chunk} slabs={slabs} weighted={weighted} acc={accumulate}", flush=True)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(ri.size).astype(np.float32) if weighted else None
    init = rng.standard_normal((Vd, F)).astype(np.float32)
    want = oracle.spmm(x, w, co, ri, Vd, fused=True) + (init if accumulate else 0)
    scale = abs_term_scale(x, w, co, ri, Vd) + (np.abs(init) if accumulate else 0)
    deg = np.diff(co.astype(np.int64))
    got = _run_planless(x, w, co, ri, Vd, F, device, accumulate=accumulate, out_init=init if accumulate else None)
    check(got, want, scale)
    if not accumulate:
        whole = deg <= (planless_piece_edges(ri.size) or ri.size + 1)
        assert np.array_equal(got[whole].view(np.uint32), want[whole].view(np.uint32))
    dx, dco, dri = _dev(x, device), _dev(co, device), _dev(ri, device)
    dw = _dev(w, device) if weighted else None
    plan = SpmmPlan(dco, Vd, ri.size, chunk, dri, Vs, slabs) if slabs > 1 else SpmmPlan(dco, Vd, ri.size, chunk)
    out = _dev(init, device) if accumulate else torch.full((Vd, F), float("nan"), device=device)
    call("nts_spmm_gather_planned", plan.handle, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, F, accumulate, _stream())
    torch.cuda.synchronize()
    got_p = out.cpu().numpy()
    check(got_p, want, scale)
    if not accumulate:
        whole = deg <= (chunk // 4 if slabs >= 8 else chunk)
        assert np.array_equal(got_p[whole].view(np.uint32), want[whole].view(np.uint32))
    plan.close()
