"""The five benchmark configurations through the host-side operator mirrors, checked against the
CPU oracle (bit-exact for index construction and gathers, max relative error <= 1e-4 in fp32 for
aggregation and edge-softmax outputs and gradients), plus size-independent properties at the full
Reddit-shaped and Products-shaped sizes."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host_u32
from neutronbench_amd import synth
from neutronbench_amd.batch import FeatureCache, MappedHostTable, load_feature_gpu_cache, load_label_gpu
from neutronbench_amd.layout import FullGraphChunk, SampledLayer, u32_to_i64
from neutronbench_amd.ops import (ForwardSingleGPUfuseOp, GATAggregateOp, GATAttentionOp, SingleGPUSampleGraphOp)
from neutronbench_amd.stream import CudaStream
from util import check

pytestmark = pytest.mark.gpu


def _scale(x, w, off, idx, rows):
    """sum of |terms| per output element, by the oracle itself on absolute values."""
    return oracle.spmm(np.abs(x), np.abs(w), off, idx, rows)


def _sample_batch(co, ri, V, batch, fanouts, seed):
    """Hops from the batch outwards, then reversed so that layer 0 is the input side
    (Sampler::sample_one, core/ntsSampler.hpp:843-1106).  Host side, oracle post-processing."""
    layers = []
    dst = batch
    for hop, fan in enumerate(fanouts):
        off, rows_global = synth.sample_hop(co, ri, dst, fan, seed + hop)
        local, source, n_src = oracle.postprocess(rows_global.numpy().astype(np.uint32), V)
        layers.append(dict(co=off.numpy().astype(np.uint32), ri=local, source=source,
                           destination=dst.numpy().astype(np.uint32)))
        dst = torch.from_numpy(source.astype(np.int64))
    return layers[::-1]


def _check_layer_structure(layer, h, V_global):
    ro_ref, ci_ref = oracle.csr_from_csc(h["co"], h["ri"], h["source"].size)
    assert np.array_equal(host_u32(layer.dev_row_offset), ro_ref)
    assert np.array_equal(host_u32(layer.dev_column_indices), ci_ref)
    outd, ind = np.ones(V_global, np.uint32), np.ones(V_global, np.uint32)
    ewf, ewb = oracle.layer_weights(h["co"], h["ri"], ro_ref, ci_ref, h["source"], h["destination"], outd, ind)
    assert layer.dev_ewf().cpu().numpy().tobytes() == ewf.tobytes()
    assert layer.dev_ewb().cpu().numpy().tobytes() == ewb.tobytes()
    return ro_ref, ci_ref, ewf, ewb


def test_config1_cora_shaped_full_graph(device):
    """2,708 nodes, 10,556 directed edges (symmetric power law), 1,433 binary features, hidden 16:
    layout bit-exact with PartitionToChunks, aggregation fwd/bwd at F=1433 and F=16."""
    V = 2708
    src, dst = synth.powerlaw_symmetric_edges(V, 5278, seed=1)
    assert src.numel() == 10556
    chunk = FullGraphChunk.from_edges(src.to(device), dst.to(device), V)
    order = np.argsort(src.numpy(), kind="stable")
    coo_s, coo_d = src.numpy()[order].astype(np.uint32), dst.numpy()[order].astype(np.uint32)
    outd, ind = oracle.degrees(coo_s, coo_d, V)
    ref = oracle.build_chunk(coo_s, coo_d, V, outd, ind)
    for name, t in (("co", chunk.column_offset_gpu), ("ri", chunk.row_indices_gpu), ("ro", chunk.row_offset_gpu),
                    ("ci", chunk.column_indices_gpu)):
        assert np.array_equal(host_u32(t), ref[name]), name
    assert chunk.edge_weight_forward_gpu.cpu().numpy().tobytes() == ref["ewf"].tobytes()
    assert chunk.edge_weight_backward_gpu.cpu().numpy().tobytes() == ref["ewb"].tobytes()
    op = ForwardSingleGPUfuseOp(chunk)
    x = synth.binary_features(V, 1433, 0.013, seed=2).numpy()
    h = np.random.default_rng(3).standard_normal((V, 16)).astype(np.float32)
    for feat in (x, h):
        d = dev(feat, device)
        y = op.forward(d).cpu().numpy()
        g = op.backward(d).cpu().numpy()
        check(y, oracle.spmm(feat, ref["ewf"], ref["co"], ref["ri"], V), _scale(feat, ref["ewf"], ref["co"], ref["ri"], V))
        check(g, oracle.spmm(feat, ref["ewb"], ref["ro"], ref["ci"], V), _scale(feat, ref["ewb"], ref["ro"], ref["ci"], V))


def test_config2_arxiv_shaped_minibatch(device):
    """169,343-node, 2.48M-edge R-MAT graph, 128 features, fanout [25,10] (the batch's own hop 25, as the
    reference's reversed FANOUT string "10,25" gives it),
    batch 1,024: sampled-layer construction bit-exact, feature/label gather bit-exact, aggregation
    forward and backward of both layers against MiniBatchFuseOp's arithmetic."""
    V, E, F = 169_343, 2_480_000, 128
    src, dst = synth.rmat_edges(V, E, seed=2)
    co, ri = synth.build_csc(src, dst, V)
    batch = synth.permutation(V, 22)[:1024]
    hops = _sample_batch(co, ri, V, batch, [25, 10], seed=22)
    feat = synth.normal_features(V, F, seed=23).numpy()
    labels = synth.uniform_labels(V, 40, seed=24).numpy()
    layers = [SampledLayer.from_host_csc(*(torch.from_numpy(h[k].astype(np.int64)) for k in
                                            ("co", "ri", "source", "destination")), device) for h in hops]
    cs = CudaStream()
    # batch assembly
    dfeat = dev(feat, device)
    x0 = torch.empty(layers[0].src_size, F, device=device)
    cs.zero_copy_feature_move_gpu(x0, dfeat, layers[0].dev_source, F, layers[0].src_size)
    assert x0.cpu().numpy().tobytes() == oracle.get_feature(feat, hops[0]["source"]).tobytes()
    dlab = dev(labels, device)
    lab = torch.empty(layers[-1].v_size, dtype=torch.int64, device=device)
    load_label_gpu(cs, layers[-1], lab, dlab)
    assert np.array_equal(lab.cpu().numpy(), oracle.get_label(labels, hops[-1]["destination"]))
    # aggregation, layer by layer (inputs: gathered features, then a seeded hidden tensor)
    x = x0
    for l, (layer, h) in enumerate(zip(layers, hops)):
        ro_ref, ci_ref, ewf, ewb = _check_layer_structure(layer, h, V)
        op = SingleGPUSampleGraphOp(layers, l, cs)
        y = op.forward(x)
        xh = x.cpu().numpy()
        check(y.cpu().numpy(), oracle.spmm(xh, ewf, h["co"], h["ri"], layer.v_size), _scale(xh, ewf, h["co"], h["ri"], layer.v_size))
        gy = synth.normal_features(layer.v_size, F, seed=30 + l, device=device)
        gx = op.backward(gy)
        gyh = gy.cpu().numpy()
        check(gx.cpu().numpy(), oracle.spmm(gyh, ewb, ro_ref, ci_ref, layer.src_size),
              _scale(gyh, ewb, ro_ref, ci_ref, layer.src_size))
        assert y.shape == (layer.v_size, F) and gx.shape == (layer.src_size, F)
        x = y  # next layer's sources are this layer's destinations
        if l + 1 < len(layers):
            assert np.array_equal(hops[l + 1]["source"], np.sort(hops[l + 1]["source"]))
            assert layers[l + 1].src_size == layer.v_size


def test_config3_reddit_shaped_full_size_properties(device):
    """232,965 nodes, 114.8M R-MAT edges resident in HBM.  At this size the checks are
    size-independent properties plus the oracle on a sample of output rows (hub rows included)."""
    V, E = 232_965, 114_800_000
    src, dst = synth.rmat_edges(V, E, seed=3, device=device)
    chunk = FullGraphChunk.from_edges(src, dst, V)
    del src, dst
    op = ForwardSingleGPUfuseOp(chunk)
    unweighted = ForwardSingleGPUfuseOp(chunk, with_weight=False)
    F = 128
    deg_in = (u32_to_i64(chunk.column_offset_gpu)[1:] - u32_to_i64(chunk.column_offset_gpu)[:-1])
    info = chunk.plan_forward.info()
    assert info["split_rows"] > 0 and int(deg_in.max()) > 100_000  # power-law hubs are present and split
    # all-ones input, unit weights -> exact in-degrees (integers below 2^24 are exact in fp32)
    ones = torch.ones(V, 8, device=device)
    got = unweighted.forward(ones)
    assert torch.equal(got, deg_in.to(torch.float32)[:, None].expand(V, 8))
    x = synth.normal_features(V, F, seed=41, device=device)
    y = synth.normal_features(V, F, seed=42, device=device)
    ax, ay, axy = op.forward(x), op.forward(y), op.forward(x + y)
    scale = op.forward(x.abs()) + op.forward(y.abs())
    lin = ((axy - (ax + ay)).abs() / torch.maximum(axy.abs(), 1e-2 * scale + 1e-30)).max().item()
    assert lin <= 1e-4, f"linearity {lin:.2e}"
    aty = op.backward(y)
    lhs = (ax.double() * y.double()).sum().item()
    rhs = (x.double() * aty.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-6 * max(abs(lhs), abs(rhs)), (lhs, rhs)
    assert torch.equal(ax, op.forward(x)) and torch.equal(aty, op.backward(y))  # bit-reproducible
    # oracle on sampled rows: 3,000 seeded random rows and the 8 largest hubs
    co = u32_to_i64(chunk.column_offset_gpu).cpu().numpy()
    xh = x.cpu().numpy()

    def sub_csc(rows):
        sub_off = np.zeros(rows.size + 1, dtype=np.uint32)
        idx_parts, w_parts = [], []
        for k, r in enumerate(rows):
            s, e = int(co[r]), int(co[r + 1])
            idx_parts.append(chunk.row_indices_gpu[s:e])
            w_parts.append(chunk.edge_weight_forward_gpu[s:e])
            sub_off[k + 1] = sub_off[k] + (e - s)
        return sub_off, host_u32(torch.cat(idx_parts)), torch.cat(w_parts).cpu().numpy()

    rows = synth.permutation(V, 5, device)[:3000].cpu().numpy()
    sub_off, sub_idx, sub_w = sub_csc(rows)
    got = ax[torch.from_numpy(rows).to(device)].cpu().numpy()
    unsplit = np.diff(sub_off.astype(np.int64)) <= 4096  # the default chunk: these rows are one FMA chain
    assert unsplit.sum() > 2000
    ref_fma = oracle.spmm(xh, sub_w, sub_off, sub_idx, rows.size, fused=True)
    assert np.array_equal(got[unsplit].view(np.uint32), ref_fma[unsplit].view(np.uint32))
    ref = oracle.spmm(xh, sub_w, sub_off, sub_idx, rows.size)
    scale = _scale(xh, sub_w, sub_off, sub_idx, rows.size)
    check(got[unsplit], ref[unsplit], scale[unsplit])
    # Hub rows (up to ~8e5 edges) are summed chunk-wise on the GPU and strictly sequentially by the
    # oracle; in fp32 the two orders legitimately differ by ~sqrt(n) ulp of the term scale, so both
    # are measured against the exact (fp64) sum: the GPU must meet the tolerance and must not be
    # less accurate than the oracle.
    hubs = torch.topk(deg_in, 8).indices.cpu().numpy()
    h_off, h_idx, h_w = sub_csc(hubs)
    got_h = ax[torch.from_numpy(hubs).to(device)].cpu().numpy()
    ref_h = oracle.spmm(xh, h_w, h_off, h_idx, hubs.size)
    scale_h = _scale(xh, h_w, h_off, h_idx, hubs.size)
    exact = np.zeros((hubs.size, F))
    for k in range(hubs.size):
        for s in range(int(h_off[k]), int(h_off[k + 1]), 1 << 16):
            e = min(s + (1 << 16), int(h_off[k + 1]))
            exact[k] += (xh[h_idx[s:e].astype(np.int64)].astype(np.float64) * h_w[s:e, None].astype(np.float64)).sum(0)
    from util import rel_err
    err_gpu = rel_err(got_h, exact, scale_h)
    err_cpu = rel_err(ref_h, exact, scale_h)
    print(f"hub rows: degrees {np.diff(h_off.astype(np.int64)).tolist()}, error vs exact: gpu {err_gpu:.2e}, cpu oracle {err_cpu:.2e}")
    assert err_gpu <= 1e-4 and err_gpu <= max(err_cpu, 1e-5)


def test_config4_products_shaped_cached_gather(device):
    """Feature gather with the HBM cache of the top-20 % out-degree nodes, rest read zero-copy from
    mapped pinned host memory.  The graph is a 1/10-scale R-MAT (245K nodes, 12.6M edges) for the
    sampled batch (6,000 nodes, fanout [15,10,5]); the gather itself is then repeated at the full
    2,449,029 x 100 table size against torch.index_select."""
    V, E, F = 244_903, 12_620_000, 100
    src, dst = synth.rmat_edges(V, E, seed=4, device=device)
    co, ri = synth.build_csc(src, dst, V)
    out_deg = torch.bincount(src, minlength=V).cpu()
    co, ri = co.cpu(), ri.cpu()
    del src, dst
    batch = synth.permutation(V, 44)[:6000]
    hops = _sample_batch(co, ri, V, batch, [15, 10, 5], seed=44)
    feat_t = synth.normal_features(V, F, seed=45)
    feat = feat_t.numpy()
    n_cache = V // 5
    table = MappedHostTable(feat_t)
    cache = FeatureCache(feat_t, out_deg, n_cache, device)
    layers = [SampledLayer.from_host_csc(*(torch.from_numpy(h[k].astype(np.int64)) for k in
                                            ("co", "ri", "source", "destination")), device) for h in hops]
    cs = CudaStream()
    src0 = hops[0]["source"]
    want = oracle.get_feature(feat, src0)
    hashmap_ref = oracle.mark_cache(V, cache.order.numpy().astype(np.uint32), n_cache)
    _, hit, miss = oracle.load_feature_cached(feat, cache.dev_cache_feature.cpu().numpy(), src0, hashmap_ref)
    x_dev_split = torch.full((src0.size, F), float("nan"), device=device)
    hits = load_feature_gpu_cache(cs, layers[0], x_dev_split, table.dev_ptr, cache)
    cs.CUDA_DEVICE_SYNCHRONIZE()
    assert x_dev_split.cpu().numpy().tobytes() == want.tobytes() and int(hits.item()) == hit.size
    x_host_split = torch.full((src0.size, F), float("nan"), device=device)
    n_hit = load_feature_gpu_cache(cs, layers[0], x_host_split, table.dev_ptr, cache,
                                   torch.from_numpy(src0.astype(np.int64)), device_split=False)
    assert x_host_split.cpu().numpy().tobytes() == want.tobytes() and n_hit == hit.size
    assert hit.size > 0.3 * src0.size  # high-degree nodes dominate sampled neighbourhoods
    # three sampled layers: structure bit-exact, aggregation within tolerance (widths 100, 128, 128)
    x = x_dev_split
    for l, (layer, h) in enumerate(zip(layers, hops)):
        ro_ref, ci_ref, ewf, ewb = _check_layer_structure(layer, h, V)
        op = SingleGPUSampleGraphOp(layers, l, cs)
        y = op.forward(x)
        xh = x.cpu().numpy()
        check(y.cpu().numpy(), oracle.spmm(xh, ewf, h["co"], h["ri"], layer.v_size), _scale(xh, ewf, h["co"], h["ri"], layer.v_size))
        gy = synth.normal_features(layer.v_size, x.shape[1], seed=50 + l, device=device)
        gx = op.backward(gy)
        gyh = gy.cpu().numpy()
        check(gx.cpu().numpy(), oracle.spmm(gyh, ewb, ro_ref, ci_ref, layer.src_size), _scale(gyh, ewb, ro_ref, ci_ref, layer.src_size))
        x = synth.normal_features(layer.v_size, 128, seed=60 + l, device=device)  # stands in for the dense layer
    table.close()
    # full-size table: 2,449,029 rows x 100 floats in mapped host memory, 1M sampled rows
    Vf = 2_449_029
    big = synth.normal_features(Vf, F, seed=46)
    big_table = MappedHostTable(big)
    ids = (synth.hash64(torch.arange(1_000_000), 99) & 0x7FFFFFFF) % Vf
    lay = SampledLayer()
    lay.src_size = ids.numel()
    lay.dev_source = ids.to(torch.int32).to(device)
    out = torch.empty(ids.numel(), F, device=device)
    cs.zero_copy_feature_move_gpu(out, big_table.dev_ptr, lay.dev_source, F, lay.src_size)
    assert torch.equal(out.cpu(), big.index_select(0, ids))
    big_table.close()


def test_config5_gat_sampled_layers(device):
    """GAT, 4 heads x 32, LeakyReLU 0.2, batch 4,096, fanout [10,10] on a 1/10-scale Products-shaped
    graph: fused attention + attention-weighted aggregation, forward and backward, against torch
    autograd (fp64) over the unfused chain index_select -> add -> leaky_relu -> per-destination
    softmax -> weighted index_add, which is the composition of the reference's CPU operators."""
    V, E, H, Fh = 244_903, 12_620_000, 4, 32
    F = H * Fh
    src, dst = synth.rmat_edges(V, E, seed=4, device=device)
    co, ri = synth.build_csc(src, dst, V)
    co, ri = co.cpu(), ri.cpu()
    del src, dst
    batch = synth.permutation(V, 55)[:4096]
    hops = _sample_batch(co, ri, V, batch, [10, 10], seed=55)
    layers = [SampledLayer.from_host_csc(*(torch.from_numpy(h[k].astype(np.int64)) for k in
                                            ("co", "ri", "source", "destination")), device) for h in hops]
    for l, (layer, h) in enumerate(zip(layers, hops)):
        Vs, Vd, Eh = layer.src_size, layer.v_size, layer.e_size
        hfeat = synth.normal_features(Vs, F, seed=70 + l, device=device)
        a_l = synth.normal_features(H, Fh, seed=80 + l, device=device) * 0.3
        a_r = synth.normal_features(H, Fh, seed=90 + l, device=device) * 0.3
        gout = synth.normal_features(Vd, F, seed=100 + l, device=device)
        # destinations of a sampled layer are not a prefix of its sources: their features are
        # looked up by global id
        src_ids = torch.from_numpy(h["source"].astype(np.int64))
        dst_ids = torch.from_numpy(h["destination"].astype(np.int64))
        pos = torch.searchsorted(src_ids, dst_ids).clamp(max=Vs - 1)
        found = (src_ids[pos] == dst_ids).to(device)
        hdst = torch.where(found[:, None], hfeat[pos.to(device)], torch.zeros(Vd, F, device=device))
        el = torch.einsum("vhf,hf->vh", hfeat.view(Vs, H, Fh), a_l).contiguous()
        er = torch.einsum("vhf,hf->vh", hdst.view(Vd, H, Fh), a_r).contiguous()
        att, agg = GATAttentionOp(layer, 0.2), GATAggregateOp(layer, H)
        alpha = att.forward(el, er)
        out = agg.forward(hfeat, alpha)
        gh = agg.backward(gout)
        galpha = agg.get_additional_grad()
        gel = att.backward(galpha)
        ger = att.get_additional_grad()
        # autograd reference in fp64
        ri_t = torch.from_numpy(h["ri"].astype(np.int64)).to(device)
        deg = np.diff(h["co"].astype(np.int64))
        dst_of = torch.from_numpy(np.repeat(np.arange(Vd), deg)).to(device)
        x64 = hfeat.double().requires_grad_(True)
        el64 = el.double().requires_grad_(True)
        er64 = er.double().requires_grad_(True)
        s = torch.nn.functional.leaky_relu(el64[ri_t] + er64[dst_of], 0.2)
        mx = torch.full((Vd, H), -float("inf"), dtype=torch.float64, device=device).index_reduce(0, dst_of, s.detach(), "amax")
        ex = torch.exp(s - mx[dst_of])
        den = torch.zeros(Vd, H, dtype=torch.float64, device=device).index_add(0, dst_of, ex)
        a64 = ex / den[dst_of]
        msg = x64[ri_t].view(Eh, H, Fh) * a64[:, :, None]
        o64 = torch.zeros(Vd, H, Fh, dtype=torch.float64, device=device).index_add(0, dst_of, msg).view(Vd, F)
        o64.backward(gout.double())
        check(alpha.cpu().numpy(), a64.detach().cpu().numpy(), scale=1.0, floor=1e-6)
        check(out.cpu().numpy(), o64.detach().cpu().numpy())
        # gradient of the features through the aggregation only (alpha held fixed) and of el / er
        x64b = hfeat.double().requires_grad_(True)
        (x64b[ri_t].view(Eh, H, Fh) * a64.detach()[:, :, None]).view(Eh, F).mul(gout.double()[dst_of]).sum().backward()
        check(gh.cpu().numpy(), x64b.grad.cpu().numpy())
        # error scale of the score gradients: every edge term alpha*(galpha - sum alpha*galpha) carries
        # the magnitude alpha*(|galpha| + sum alpha*|galpha|); el / er gradients add those terms up
        ga = galpha.double().abs()
        a_det = a64.detach()
        seg = torch.zeros(Vd, H, dtype=torch.float64, device=device).index_add(0, dst_of, a_det * ga)
        term = a_det * (ga + seg[dst_of])
        s_el = torch.zeros(Vs, H, dtype=torch.float64, device=device).index_add(0, ri_t, term)
        s_er = torch.zeros(Vd, H, dtype=torch.float64, device=device).index_add(0, dst_of, term)
        check(gel.cpu().numpy(), el64.grad.cpu().numpy(), scale=s_el.cpu().numpy())
        check(ger.cpu().numpy(), er64.grad.cpu().numpy(), scale=s_er.cpu().numpy())
