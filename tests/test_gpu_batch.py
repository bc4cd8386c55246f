"""GPU parity of mini-batch assembly (feature / label gather, HBM feature cache, zero-copy reads of
mapped pinned host memory) and of the device-side sampled-layer construction: bit-exact."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host_u32, stream
from neutronbench_amd import abi
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.batch import (FeatureCache, MappedHostTable, load_feature_gpu, load_feature_gpu_cache,
                                    load_label_gpu, sample_hop)
from neutronbench_amd.layout import SampledLayer, as_u32
from neutronbench_amd.stream import CudaStream, get_gpu_mem
from util import brute_csr, random_block

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("F", [1, 3, 8, 100, 128, 602, 1433])
def test_feature_gather_device_table(device, F):
    print(f"case F={F}", flush=True)
    rng = np.random.default_rng(F)
    V, n = 3000, 1111
    feat = rng.standard_normal((V, F)).astype(np.float32)
    ids = rng.integers(0, V, n).astype(np.uint32)
    out = torch.full((n, F), float("nan"), device=device)
    dfeat, dids = dev(feat, device), dev(ids, device)  # keep the device copies alive across the call
    call("nts_gather_rows_f32", ptr(out), ptr(dfeat), ptr(dids), 0, 0, n, F, stream())
    assert out.cpu().numpy().tobytes() == oracle.get_feature(feat, ids).tobytes()


def test_feature_gather_zero_copy_and_cache(device):
    """The three launches of the reference (plain zero-copy, zero-copy of the miss list, cache
    gather of the hit list) and the single device-split kernel all reproduce get_feature."""
    rng = np.random.default_rng(1)
    V, F, n_cache = 5000, 100, 1000
    feat = rng.standard_normal((V, F)).astype(np.float32)
    out_deg = rng.integers(0, 200, V)
    feat_t = torch.from_numpy(feat)
    table = MappedHostTable(feat_t)
    cache = FeatureCache(feat_t, torch.from_numpy(out_deg), n_cache, device)
    order = cache.order.numpy().astype(np.uint32)
    hashmap_ref = oracle.mark_cache(V, order, n_cache)
    assert np.array_equal(cache.cache_node_hashmap.numpy().view(np.uint32), hashmap_ref)
    assert np.array_equal(cache.dev_cache_feature.cpu().numpy(), oracle.fill_cache(feat, order, n_cache, hashmap_ref))

    source = np.sort(rng.choice(V, 1800, replace=False)).astype(np.uint32)
    layer0 = SampledLayer()
    layer0.src_size = source.size
    layer0.dev_source = dev(source, device)
    cs = CudaStream()
    want, hit, miss = oracle.load_feature_cached(feat, cache.dev_cache_feature.cpu().numpy(), source, hashmap_ref)
    assert want.tobytes() == oracle.get_feature(feat, source).tobytes()

    x0 = torch.full((source.size, F), float("nan"), device=device)
    load_feature_gpu(cs, layer0, x0, table.dev_ptr)
    assert x0.cpu().numpy().tobytes() == want.tobytes()

    x1 = torch.full((source.size, F), float("nan"), device=device)
    n_hit = load_feature_gpu_cache(cs, layer0, x1, table.dev_ptr, cache, torch.from_numpy(source.astype(np.int64)),
                                   device_split=False)
    assert n_hit == hit.size and x1.cpu().numpy().tobytes() == want.tobytes()

    x2 = torch.full((source.size, F), float("nan"), device=device)
    hits = load_feature_gpu_cache(cs, layer0, x2, table.dev_ptr, cache)
    cs.CUDA_DEVICE_SYNCHRONIZE()
    assert int(hits.item()) == hit.size and x2.cpu().numpy().tobytes() == want.tobytes()
    table.close()


def test_label_gather(device):
    rng = np.random.default_rng(2)
    V, n = 4000, 1024
    ids = rng.integers(0, V, n).astype(np.uint32)
    top = SampledLayer()
    top.v_size = n
    top.dev_destination = dev(ids, device)
    cs = CudaStream()
    lab = rng.integers(0, 47, V).astype(np.int64)
    out = torch.full((n,), -1, dtype=torch.int64, device=device)
    dlab = dev(lab, device)
    load_label_gpu(cs, top, out, dlab)
    assert np.array_equal(out.cpu().numpy(), oracle.get_label(lab, ids))
    multi = rng.integers(0, 2, (V, 121)).astype(np.int64)
    out2 = torch.full((n, 121), -1, dtype=torch.int64, device=device)
    dmulti = dev(multi, device)
    load_label_gpu(cs, top, out2, dmulti)
    assert np.array_equal(out2.cpu().numpy(), oracle.get_label(multi, ids))


@pytest.mark.parametrize("Vd,Vs,mean,hub,dup", [(1024, 9000, 12, 0, False), (300, 50, 20, 45, False),
                                                (2000, 700, 6, 5000, True), (1, 1, 1, 0, False)])
def test_device_csr_and_weights(device, Vd, Vs, mean, hub, dup):
    """generate_csr_from_csc + update_degree + compute_weight_* on the device are bit-exact with
    the host algorithms of the oracle."""
    print(f"case Vd={Vd} Vs={Vs}", flush=True)
    co, ri = random_block(Vd, Vs, mean, seed=Vd + Vs, hub=hub, dup=dup, empty_frac=0.05)
    E = ri.size
    rng = np.random.default_rng(3)
    V = 20000
    glob = rng.permutation(V)
    source = np.sort(glob[:Vs]).astype(np.uint32)
    destination = glob[Vs:Vs + Vd].astype(np.uint32)
    layer = SampledLayer.from_host_csc(torch.from_numpy(co.astype(np.int64)), torch.from_numpy(ri.astype(np.int64)),
                                       torch.from_numpy(source.astype(np.int64)),
                                       torch.from_numpy(destination.astype(np.int64)), device)
    torch.cuda.synchronize()
    ro_ref, ci_ref = oracle.csr_from_csc(co, ri, Vs)
    assert np.array_equal(host_u32(layer.dev_row_offset), ro_ref)
    assert np.array_equal(host_u32(layer.dev_column_indices), ci_ref)
    _, _, perm = brute_csr(co, ri, Vs)
    assert np.array_equal(host_u32(layer.dev_csr_to_csc), perm)
    outd = np.ones(V, np.uint32)
    ind = np.ones(V, np.uint32)
    ewf_ref, ewb_ref = oracle.layer_weights(co, ri, ro_ref, ci_ref, source, destination, outd, ind)
    assert layer.dev_ewf().cpu().numpy().tobytes() == ewf_ref.tobytes()
    assert layer.dev_ewb().cpu().numpy().tobytes() == ewb_ref.tobytes()
    assert np.array_equal(host_u32(layer.dev_source), source) and np.array_equal(host_u32(layer.dev_destination), destination)


def test_norm_weight_table_bit_exact(device):
    """Every (out_degree, in_degree) pair up to 64 x 64 through the device weight kernel equals
    nts_norm_degree bit for bit: a star per source degree."""
    n = 64
    # destination d (1-based degree) gets d in-edges; source s gets s out-edges: build a complete
    # bipartite-like block where source j connects to destinations j..n-1 -> out_deg(j) = n-j,
    # in_deg(d) = d+1
    co = np.zeros(n + 1, dtype=np.uint32)
    ri = []
    for d in range(n):
        ri += list(range(0, d + 1))
        co[d + 1] = len(ri)
    ri = np.array(ri, dtype=np.uint32)
    ro, ci, perm = brute_csr(co, ri, n)
    ewf = torch.empty(ri.size, device=device)
    ewb = torch.empty(ri.size, device=device)
    dco, dri, dro, dci = (dev(t, device) for t in (co, ri, ro, ci))
    call("nts_gcn_edge_weights", ptr(ewf), ptr(ewb), ptr(dco), ptr(dri), ptr(dro), ptr(dci), n, n, stream())
    got = ewf.cpu().numpy()
    k = 0
    for d in range(n):
        for s in range(d + 1):
            assert got[k].tobytes() == oracle.norm_degree(n - s, d + 1).tobytes(), (s, d)
            k += 1
    assert np.array_equal(ewb.cpu().numpy(), got[perm])


def test_memory_and_stream_entry_points(device):
    used, total = get_gpu_mem()
    assert 0 <= used <= total and total > 64 * 1024  # MiB: an MI355X has far more than 64 GiB
    p = ctypes.c_void_p()
    call("nts_malloc_device", ctypes.byref(p), 1 << 20)
    assert p.value
    s = ctypes.c_void_p()
    call("nts_stream_create", ctypes.byref(s))
    host = np.arange(1 << 18, dtype=np.uint32)
    back = np.zeros_like(host)
    call("nts_memcpy_h2d_async", p, host.ctypes.data, host.nbytes, s)
    call("nts_memcpy_d2h_async", back.ctypes.data, p, host.nbytes, s)
    call("nts_stream_sync", s)
    assert np.array_equal(host, back)
    # unaligned, odd-sized zero fill touches exactly the requested bytes
    call("nts_memcpy_h2d", p, host.ctypes.data, host.nbytes, 1)
    call("nts_memset_zero", p.value + 3, 1001, s)
    call("nts_memcpy_d2h_async", back.ctypes.data, p, host.nbytes, s)
    call("nts_stream_sync", s)
    want = host.copy().view(np.uint8)
    want[3:1004] = 0
    assert np.array_equal(back.view(np.uint8), want)
    q = ctypes.c_void_p()
    call("nts_malloc_device_async", ctypes.byref(q), 4096, s)
    call("nts_free_device_async", q, s)
    call("nts_stream_sync", s)
    call("nts_stream_destroy", s)
    call("nts_free_device", p)
    hp, dp = ctypes.c_void_p(), ctypes.c_void_p()
    call("nts_malloc_pinned_mapped", ctypes.byref(hp), 4096)
    call("nts_host_get_device_ptr", ctypes.byref(dp), hp)
    assert dp.value
    call("nts_free_pinned", hp)
    assert abi.status("nts_memcpy_h2d", 0, host.ctypes.data, 16, 0) == abi.NTS_ERR_INVALID


@pytest.mark.parametrize("V,E,seed", [(5000, 3000, 1), (100, 50000, 2), (1 << 16, 200000, 3), (37, 1, 4)])
def test_device_relabel_matches_host_bitmap_scan(device, V, E, seed):
    """sampCSC::postprocessing on the device: sorted distinct sources and local ids, bit-exact."""
    rng = np.random.default_rng(seed)
    glob = rng.integers(0, V, E).astype(np.uint32)
    glob[0] = V - 1
    want_local, want_source, n = oracle.postprocess(glob, V)
    dglob = dev(glob, device)
    work = torch.empty(call("nts_relabel_sources_work_bytes", V) + 256, dtype=torch.uint8, device=device)
    base = (work.data_ptr() + 255) // 256 * 256
    source = torch.full((max(min(E, V), 1),), -1, dtype=torch.int32, device=device)
    n_source = torch.zeros(1, dtype=torch.int32, device=device)
    local = torch.empty(E, dtype=torch.int32, device=device)
    call("nts_relabel_sources", ptr(source), ptr(n_source), ptr(local), ptr(dglob), E, V, base, stream())
    assert int(n_source.item()) == n
    assert np.array_equal(host_u32(source[:n]), want_source)
    assert np.array_equal(host_u32(local), want_local)


def test_fully_device_side_layer_construction(device):
    """Hop sampled on the device -> relabel -> CSR -> weights, no host step: equal to the host
    pipeline of the oracle (postprocessing, generate_csr_from_csc, update_degree + weights)."""
    from neutronbench_amd import synth
    from neutronbench_amd.layout import as_u32

    V, E = 30000, 600000
    src, dst = synth.rmat_edges(V, E, seed=8, device=device, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    batch = synth.permutation(V, 9, device)[:2000]
    off, rows_global = synth.sample_hop(co, ri, batch, 10, 3)
    layer = SampledLayer.from_device_hop(as_u32(off), as_u32(rows_global), as_u32(batch), V)
    torch.cuda.synchronize()
    glob = rows_global.cpu().numpy().astype(np.uint32)
    local, source, n = oracle.postprocess(glob, V)
    co_h = off.cpu().numpy().astype(np.uint32)
    assert layer.src_size == n and np.array_equal(host_u32(layer.dev_source), source)
    assert np.array_equal(host_u32(layer.dev_row_indices), local)
    ro_ref, ci_ref = oracle.csr_from_csc(co_h, local, n)
    assert np.array_equal(host_u32(layer.dev_row_offset), ro_ref) and np.array_equal(host_u32(layer.dev_column_indices), ci_ref)
    outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
    ewf, ewb = oracle.layer_weights(co_h, local, ro_ref, ci_ref, source, batch.cpu().numpy().astype(np.uint32), outd, ind)
    assert layer.dev_ewf().cpu().numpy().tobytes() == ewf.tobytes() and layer.dev_ewb().cpu().numpy().tobytes() == ewb.tobytes()


@pytest.mark.parametrize("fanout", [-1, 1, 5, 25, 64, 65, 100, 700])
def test_device_sampler_properties(device, fanout):
    """The hop sampler's contract: offsets equal init_co (bit-exact); with nothing dropped a
    destination's neighbours come out in CSC order; otherwise `fanout` DISTINCT positions of its
    segment, ascending; the same seed reproduces the sample and another seed changes it.  These are
    the reference's own validity conditions (Sampler::isValidSampleGraph / sample_one asserts)."""
    from neutronbench_amd import synth
    from neutronbench_amd.layout import as_u32

    V, E = 20000, 600000
    src, dst = synth.rmat_edges(V, E, seed=12, device=device, sort=True)
    co64, ri64 = synth.build_csc(src, dst, V)
    gco, gri = as_u32(co64), as_u32(ri64)
    batch64 = synth.permutation(V, 13, device)[:3000]
    batch = as_u32(batch64)
    co, ri = sample_hop(gco, gri, batch, fanout, 77)
    torch.cuda.synchronize()
    co_h = host_u32(co)
    assert np.array_equal(co_h, oracle.init_co(co64.cpu().numpy().astype(np.uint32), batch64.cpu().numpy().astype(np.uint32), fanout))
    ri_h = host_u32(ri)
    gco_h, gri_h = co64.cpu().numpy(), ri64.cpu().numpy()
    b = batch64.cpu().numpy()
    partial_rows = 0
    for i in range(b.size):
        seg = gri_h[gco_h[b[i]]:gco_h[b[i] + 1]]
        got = ri_h[co_h[i]:co_h[i + 1]]
        if got.size == seg.size:
            assert np.array_equal(got, seg)
            continue
        partial_rows += 1
        assert got.size == fanout
        # distinct positions, ascending: `got` must be a subsequence of the (sorted, duplicates kept) segment
        pos, ok = 0, True
        for v in got:
            while pos < seg.size and seg[pos] != v:
                pos += 1
            ok = ok and pos < seg.size
            pos += 1
        assert ok, f"destination slot {i}: not {fanout} distinct positions of its neighbour list"
    if 0 < fanout < 100:
        assert partial_rows > 0
    co2, ri2 = sample_hop(gco, gri, batch, fanout, 77)
    assert torch.equal(ri, ri2) and torch.equal(co, co2)
    if partial_rows:
        _, ri3 = sample_hop(gco, gri, batch, fanout, 78)
        assert not torch.equal(ri, ri3)


def test_device_sampler_is_uniform(device):
    """Every position of a long neighbour list is picked about equally often (fanout 8 of 64)."""
    deg, n, fanout = 64, 20000, 8
    gco = torch.tensor([0, deg], dtype=torch.int32, device=device)
    gri = torch.arange(deg, dtype=torch.int32, device=device)
    dst = torch.zeros(n, dtype=torch.int32, device=device)
    co, ri = sample_hop(gco, gri, dst, fanout, 5)
    counts = torch.bincount(ri.to(torch.int64), minlength=deg).cpu().numpy()
    expect = n * fanout / deg
    assert counts.sum() == n * fanout
    assert np.all(np.abs(counts - expect) < 6 * np.sqrt(expect)), counts


def test_wide_fanouts_pick_spread_positions_uniformly(device):
    """Fanouts above one wavefront (65 .. 1,024) take their positions from a keyed permutation of the
    neighbourhood: every position about equally often, and the picks of one destination are spread
    over the whole list instead of forming a run of neighbouring positions."""
    deg, n, fanout = 1000, 4000, 100
    gco = torch.tensor([0, deg], dtype=torch.int32, device=device)
    gri = torch.arange(deg, dtype=torch.int32, device=device)
    dst = torch.zeros(n, dtype=torch.int32, device=device)
    co, ri = sample_hop(gco, gri, dst, fanout, 9)
    picks = ri.cpu().numpy().reshape(n, fanout)
    assert all(np.unique(row).size == fanout for row in picks[:200])
    assert np.all(np.diff(picks, axis=1) > 0)  # ascending inside a destination
    counts = np.bincount(picks.ravel(), minlength=deg)
    expect = n * fanout / deg
    assert np.all(np.abs(counts - expect) < 6 * np.sqrt(expect)), (counts.min(), counts.max(), expect)
    # a window of consecutive positions would give a span of about `fanout`; spread picks span nearly the list
    spans = picks[:, -1] - picks[:, 0]
    assert np.median(spans) > 0.9 * deg
    # pairs of positions are not tied together: positions 0 and 1 are picked together about (fanout/deg)^2 of the time
    both = np.mean((picks == 0).any(1) & (picks == 1).any(1))
    assert both < 3 * (fanout / deg) ** 2 + 0.01


@pytest.mark.parametrize("deg,fanout,n", [(20000, 1500, 300), (70001, 5000, 60), (1025, 1025, 8), (1100, 1025, 200)])
def test_fanouts_above_1024_pick_the_smallest_keyed_hashes(device, deg, fanout, n):
    """Any larger fanout (the reference's sampler takes any, core/ntsSampler.hpp:936-1042): the positions
    with the `fanout` smallest keyed hashes, found by a radix select -- exactly `fanout` distinct positions
    of the neighbourhood in ascending order, every position about equally often, the same picks for the
    same seed; destinations with at most `fanout` neighbours keep all of them in CSC order."""
    small = 700  # a second vertex with fewer neighbours than the fanout
    gco = torch.tensor([0, deg, deg + small], dtype=torch.int32, device=device)
    gri = torch.cat([torch.arange(deg, dtype=torch.int32), 5 * torch.arange(small, dtype=torch.int32)]).to(device)
    dst = torch.zeros(n + 1, dtype=torch.int32, device=device)
    dst[n] = 1
    co, ri = sample_hop(gco, gri, dst, fanout, 21)
    take = min(deg, fanout)
    assert int(co[-1]) == n * take + small
    flat = ri.cpu().numpy()
    assert np.array_equal(flat[n * take:], 5 * np.arange(small))
    picks = flat[:n * take].reshape(n, take)
    assert picks.min() >= 0 and picks.max() < deg
    assert np.all(np.diff(picks, axis=1) > 0)  # ascending, hence distinct
    if take < deg:
        counts = np.bincount(picks.ravel(), minlength=deg)
        expect = n * take / deg
        assert np.all(np.abs(counts - expect) < 6 * np.sqrt(expect) + 1), (counts.min(), counts.max(), expect)
        assert np.unique(picks, axis=0).shape[0] > n // 2  # destinations do not share one sample
        co2, ri2 = sample_hop(gco, gri, dst, fanout, 21)
        assert torch.equal(ri, ri2)
        _, ri3 = sample_hop(gco, gri, dst, fanout, 22)
        assert not torch.equal(ri, ri3)


def test_batch_builder_with_a_fanout_above_1024(device):
    """The whole-batch builder with a hop of fanout 2,000 on a graph with a 6,000-neighbour hub: layers
    equal to the per-hop entry points, the hub's destination keeps 2,000 distinct neighbours."""
    from neutronbench_amd.batch import BatchBuilder

    V = 8000
    rng = np.random.default_rng(4)
    deg = rng.integers(1, 30, V)
    deg[17] = 6000
    gco_h = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    gri_h = np.concatenate([np.sort(rng.choice(V, d, replace=False)) for d in deg]).astype(np.int64)
    gco = as_u32(torch.from_numpy(gco_h)).to(device)
    gri = as_u32(torch.from_numpy(gri_h)).to(device)
    batch = as_u32(torch.tensor([17, 5, 900, 17], dtype=torch.int64)).to(device)
    builder = BatchBuilder(gco, gri, [2000, 3], 16)
    layers = builder.sample(batch, 99)
    top = layers[-1]
    co = top.dev_column_offset.cpu().numpy()
    assert co[1] - co[0] == 2000 and co[4] - co[3] == 2000 and co[2] - co[1] == deg[5]
    src = top.dev_source.cpu().numpy()
    local = top.dev_row_indices.cpu().numpy()[co[0]:co[1]]
    glob = src[local]
    assert np.unique(glob).size == 2000 and np.all(np.isin(glob, gri_h[gco_h[17]:gco_h[18]]))
    off, rows = sample_hop(gco, gri, batch, 2000, 99)
    assert np.array_equal(off.cpu().numpy(), co)
    assert np.array_equal(np.sort(np.unique(rows.cpu().numpy())), src)
    builder.close()


@pytest.mark.parametrize("Vs,E,skew", [
    (1, 5000, 0.0),            # one source: every key equal, one digit, one pass
    (700, 2047, 0.0),          # one edge short of a chunk
    (1024, 2048, 0.5),         # exactly one chunk, ten key bits: one pass
    (1025, 2049, 0.5),         # eleven key bits: two passes; one edge into the second chunk
    (40000, 100_000, 0.9),     # sixteen bits, a hub source holding most edges
    (1_100_000, 300_000, 0.3), # twenty-one bits: three passes, most sources without an edge
    (3_000_000, 70_000, 0.0),  # twenty-two bits
])
def test_hop_sort_over_digit_widths_and_chunk_boundaries(device, Vs, E, skew):
    """nts_csr_from_csc sorts (local source, CSC edge id) with the library's own radix sort: passes of
    equal width over ceil(bits / 10) digits, 2,048 edges per block.  Against numpy's stable sort, for
    key widths that take one to three passes, edge counts on both sides of a chunk boundary, equal
    keys in bulk (stability) and sparse keys."""
    rng = np.random.default_rng(Vs + E)
    Vd = max(1, E // 7)
    cuts = np.sort(rng.integers(0, E + 1, Vd - 1))
    co = np.concatenate([[0], cuts, [E]]).astype(np.uint32)
    ri = rng.integers(0, Vs, E).astype(np.uint32)
    if skew:
        hub = rng.integers(0, Vs)
        ri[rng.random(E) < skew] = hub
    order = np.argsort(ri, kind="stable").astype(np.uint32)
    ro_want = np.searchsorted(ri[order], np.arange(Vs + 1)).astype(np.uint32)
    owner = (np.searchsorted(co, np.arange(E), side="right") - 1).astype(np.uint32)
    ci_want = owner[order]
    d_co, d_ri = torch.from_numpy(co.view(np.int32)).to(device), torch.from_numpy(ri.view(np.int32)).to(device)
    ro = torch.empty(Vs + 1, dtype=torch.int32, device=device)
    ci = torch.empty(E, dtype=torch.int32, device=device)
    perm = torch.empty(E, dtype=torch.int32, device=device)
    nbytes = call("nts_csr_from_csc_work_bytes", Vd, Vs, E)
    work = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
    base = (work.data_ptr() + 255) // 256 * 256
    s = torch.cuda.current_stream().cuda_stream
    for with_perm in (True, False):
        ro.fill_(-1)
        ci.fill_(-1)
        call("nts_csr_from_csc", ptr(ro), ptr(ci), ptr(perm) if with_perm else 0, ptr(d_co), ptr(d_ri), Vd, Vs, E, base, s)
        torch.cuda.synchronize()
        assert np.array_equal(host_u32(ro), ro_want)
        assert np.array_equal(host_u32(ci), ci_want)
        if with_perm:
            assert np.array_equal(host_u32(perm), order)
