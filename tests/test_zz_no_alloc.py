"""nts_spmm_gather_static_scratch (the aggregation entry point that allocates nothing) against
nts_spmm_gather, through the C ABI.

Both run the same kernels over the same pieces, so their outputs must be bit-identical; the oracle is
the second witness (1e-4 relative in fp32, the tolerance of the aggregation tests).  Two calls in a
row share the fixed scratch: a large block first, then a smaller one whose pieces land in memory the
first call has used.  Requests beyond the fixed size are refused before any launch.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, stream
from neutronbench_amd import abi
from neutronbench_amd.abi import call, ptr
from util import check

pytestmark = pytest.mark.gpu


def _block(Vd, Vs, mean_deg, hubs, seed):
    """Bipartite CSC block with duplicates allowed: Poisson degrees plus a few hub rows, so that
    rows on both sides of the 256-edge piece length occur."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(mean_deg, Vd).astype(np.int64)
    deg[rng.random(Vd) < 0.05] = 0
    for k, h in enumerate(hubs):
        deg[(k * 7919) % Vd] = h
    co = np.zeros(Vd + 1, dtype=np.int64)
    co[1:] = np.cumsum(deg)
    ri = rng.integers(0, Vs, int(co[-1]))
    return co.astype(np.uint32), ri.astype(np.uint32)


def _both(device, Vd, Vs, F, mean_deg, hubs, seed, accumulate=0):
    co, ri = _block(Vd, Vs, mean_deg, hubs, seed)
    E = ri.size
    print(f"case Vd={Vd} Vs={Vs} F={F} E={E} hubs={hubs} seed={seed} accumulate={accumulate}", flush=True)
    rng = np.random.default_rng(seed + 1)
    x = rng.standard_normal((Vs, F)).astype(np.float32)
    w = rng.random(E).astype(np.float32)
    init = rng.standard_normal((Vd, F)).astype(np.float32)
    dx, dw, dco, dri = dev(x, device), dev(w, device), dev(co, device), dev(ri, device)
    outs = []
    for name in ("nts_spmm_gather", "nts_spmm_gather_static_scratch"):
        out = dev(init, device) if accumulate else torch.full((Vd, F), float("nan"), device=device)
        torch.cuda.synchronize()
        blocks_before = call("nts_scratch_alloc_count")
        free_before = torch.cuda.mem_get_info()[0]
        call(name, ptr(dx), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, Vd, E, F, accumulate, stream())
        torch.cuda.synchronize()
        if name == "nts_spmm_gather_static_scratch":
            # the property the entry point exists for: no scratch block taken, no device memory gone
            assert call("nts_scratch_alloc_count") == blocks_before
            assert torch.cuda.mem_get_info()[0] == free_before
        elif E >= 65536:
            assert call("nts_scratch_alloc_count") > blocks_before  # the pooled path does take scratch here
        outs.append(out.cpu().numpy())
    pooled, fixed = outs
    assert np.array_equal(pooled.view(np.uint32), fixed.view(np.uint32)), "static-scratch result differs"
    return fixed, (x, w, co, ri, init)


def test_two_calls_in_a_row_second_smaller(device):
    # 1st: ~1.3 M edges (ordered pieces are skipped below 2^22 edges; hub rows are cut into pieces)
    got, (x, w, co, ri, _) = _both(device, 20000, 30000, 128, 60, [70000, 9000, 3000, 700, 257, 256], seed=1)
    sample = np.unique(np.concatenate([np.arange(0, 20000, 97), np.nonzero(np.diff(co.astype(np.int64)) > 256)[0]]))
    sub_co = np.zeros(sample.size + 1, dtype=np.int64)
    sub_co[1:] = np.cumsum(np.diff(co.astype(np.int64))[sample])
    sub_ri = np.concatenate([ri[co[r]:co[r + 1]] for r in sample])
    sub_w = np.concatenate([w[co[r]:co[r + 1]] for r in sample])
    ref = oracle.spmm(x, sub_w, sub_co.astype(np.uint32), sub_ri, sample.size)
    scale = oracle.spmm(np.abs(x), sub_w, sub_co.astype(np.uint32), sub_ri, sample.size)
    check(got[sample], ref, scale)
    # 2nd, smaller, on the scratch the first call left behind; odd width (4-byte lanes), accumulate
    got2, (x2, w2, co2, ri2, init2) = _both(device, 3000, 5000, 75, 30, [5000, 300], seed=2, accumulate=1)
    ref2 = oracle.spmm(x2, w2, co2, ri2, 3000) + init2
    scale2 = oracle.spmm(np.abs(x2), w2, co2, ri2, 3000) + np.abs(init2)
    check(got2, ref2, scale2)
    # 3rd: below 65,536 edges no scratch is used at all
    got3, (x3, w3, co3, ri3, _) = _both(device, 500, 800, 602, 20, [900], seed=3)
    assert np.array_equal(got3.view(np.uint32), oracle.spmm(x3, w3, co3, ri3, 500, fused=True).view(np.uint32))


def test_large_call_with_ordered_pieces(device):
    """From 2^22 edges up the pieces are also ordered by source (a sort inside the fixed scratch)."""
    got, (x, w, co, ri, _) = _both(device, 60000, 50000, 32, 75, [200000, 40000], seed=4)
    assert ri.size >= 1 << 22
    rows = np.concatenate([np.arange(0, 60000, 601), np.nonzero(np.diff(co.astype(np.int64)) > 30000)[0]])
    sub_co = np.zeros(rows.size + 1, dtype=np.int64)
    sub_co[1:] = np.cumsum(np.diff(co.astype(np.int64))[rows])
    sub_ri = np.concatenate([ri[co[r]:co[r + 1]] for r in rows])
    sub_w = np.concatenate([w[co[r]:co[r + 1]] for r in rows])
    ref = oracle.spmm(x, sub_w, sub_co.astype(np.uint32), sub_ri, rows.size)
    scale = oracle.spmm(np.abs(x), sub_w, sub_co.astype(np.uint32), sub_ri, rows.size)
    check(got[rows], ref, scale)


def test_request_beyond_the_fixed_scratch_is_refused(device):
    """A call whose pieces would not fit is rejected with both sizes in the message and launches
    nothing (the output keeps its contents)."""
    Vd, F = 1000, 602
    E = 40_000_000  # pieces alone: (E/256 + 1000 + 1) * 602 * 4 bytes = 379 MB > 64 MiB
    co = torch.zeros(Vd + 1, dtype=torch.int32, device=device)
    out = torch.full((Vd, F), 7.0, device=device)
    dummy = torch.zeros(16, device=device)
    rc = abi.status("nts_spmm_gather_static_scratch", ptr(dummy), ptr(out), 0, ptr(co), ptr(co), 0, Vd, E, F, 0,
                    stream())
    assert rc == abi.NTS_ERR_INVALID
    msg = abi.last_error()
    assert "fixed scratch holds 67108864" in msg and "needs" in msg, msg
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())


def test_static_scratch_call_recorded_into_a_hip_graph(device):
    """The use the entry point is advertised for: a call recorded into a HIP graph (kernel launches
    only) and replayed with new inputs, eager work and synchronisations in between; every replay equals
    nts_spmm_gather on the same inputs bit for bit."""
    Vd, Vs, F = 20000, 30000, 64
    co, ri = _block(Vd, Vs, 40, [50000, 4000, 300], seed=7)
    E = ri.size
    assert 65536 <= E < (1 << 22)
    rng = np.random.default_rng(8)
    dw, dco, dri = dev(rng.random(E).astype(np.float32), device), dev(co, device), dev(ri, device)
    x = torch.zeros(Vs, F, device=device)
    out = torch.zeros(Vd, F, device=device)
    ref = torch.zeros(Vd, F, device=device)

    def run(stream_handle):
        call("nts_spmm_gather_static_scratch", ptr(x), ptr(out), ptr(dw), ptr(dco), ptr(dri), 0, Vd, E, F, 0,
             stream_handle)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(side.cuda_stream)  # the first call on a device looks the scratch address up: before the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    blocks_before = call("nts_scratch_alloc_count")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(torch.cuda.current_stream().cuda_stream)
    for rep in range(4):
        x.copy_(torch.from_numpy(rng.standard_normal((Vs, F)).astype(np.float32)))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        call("nts_spmm_gather", ptr(x), ptr(ref), ptr(dw), ptr(dco), ptr(dri), 0, Vd, E, F, 0, stream())
        torch.cuda.synchronize()
        assert torch.equal(got, ref), f"replay {rep} differs from nts_spmm_gather"
        assert float(ref.abs().sum()) > 0
    # nothing but the comparison calls took scratch
    assert call("nts_scratch_alloc_count") == blocks_before + 4
