"""Configurations 3, 4 and 5 at their stated sizes, through the entry points the benchmarks time,
against the CPU oracle.

Config 3 is built exactly as bench.py builds it (edge list in (source, destination) order, cache-aware
schedule with 512-edge pieces and 32 source ranges) and checked at F=602 and F=128, forward and
backward, on seeded rows of every schedule class: rows that are never cut (at most 128 edges; bit for
bit against the oracle's fused chain), rows that may be cut at the wide source ranges (129..512 edges)
and rows cut into pieces (longer), the largest hubs against an fp64 sum as well.
Configs 4 and 5 run one batch on the whole 2,449,029-vertex / 126.2 M-edge graph: layer construction
and gathers bit for bit, aggregation, attention and softmax within 1e-4 (fp32), and the full-graph
edge softmax / fused attention on sampled destination segments that include the largest hub.
"""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import host_u32, stream
from neutronbench_amd import synth
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.batch import BatchBuilder, FeatureCache, MappedHostTable, load_feature_gpu_cache, load_label_gpu
from neutronbench_amd.epoch import CONFIGS
from neutronbench_amd.layout import FullGraphChunk, as_u32, u32_to_i64
from neutronbench_amd.ops import ForwardSingleGPUfuseOp, GATAggregateOp, GATAttentionOp, SingleGPUSampleGraphOp
from neutronbench_amd.stream import CudaStream
from util import check, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


def sub_segments(off64, rows):
    """Edge positions of the listed rows, row after row: (sub offsets [n+1] host uint32, edge ids
    int64 on the device of `off64`)."""
    starts = off64[rows]
    lens = off64[rows + 1] - starts
    sub = torch.zeros(rows.numel() + 1, dtype=torch.int64, device=off64.device)
    sub[1:] = torch.cumsum(lens, 0)
    eid = torch.repeat_interleave(starts - sub[:-1], lens) + torch.arange(int(sub[-1]), device=off64.device)
    return sub.cpu().numpy().astype(np.uint32), eid


def exact_rows_f64(x, idx64, w, sub_off):
    """sum_e w[e] * x[idx[e], :] per row in float64 on the device (chunks of 32,768 edges)."""
    out = torch.zeros(sub_off.size - 1, x.shape[1], dtype=torch.float64, device=x.device)
    for k in range(sub_off.size - 1):
        for s in range(int(sub_off[k]), int(sub_off[k + 1]), 1 << 15):
            e = min(s + (1 << 15), int(sub_off[k + 1]))
            out[k] += (x[idx64[s:e]].double() * w[s:e, None].double()).sum(0)
    return out.cpu().numpy()


def check_aggregation_rows(tag, out, x, xh, off_dev, idx_dev, w_dev, rows, hubs, whole_limit):
    """Sampled rows of one aggregation pass against the oracle; returns the class counts."""
    off64 = u32_to_i64(off_dev)
    rows_d = torch.from_numpy(rows).to(out.device)
    sub_off, eid = sub_segments(off64, rows_d)
    sub_idx = host_u32(idx_dev[eid])
    sub_w = w_dev[eid].cpu().numpy()
    got = out[rows_d].cpu().numpy()
    deg = np.diff(sub_off.astype(np.int64))
    whole = deg <= whole_limit
    ref_fma = oracle.spmm(xh, sub_w, sub_off, sub_idx, rows.size, fused=True)
    assert np.array_equal(got[whole].view(np.uint32), ref_fma[whole].view(np.uint32)), f"{tag}: uncut rows differ"
    ref = oracle.spmm(xh, sub_w, sub_off, sub_idx, rows.size)
    scale = oracle.spmm(np.abs(xh), sub_w, sub_off, sub_idx, rows.size)
    err = rel_err(got, ref, scale)
    assert err <= TOL, f"{tag}: sampled rows, max relative error {err:.3e}"
    # the largest hubs: chunked on the GPU, strictly sequential in the oracle; both against fp64
    hubs_d = torch.from_numpy(hubs).to(out.device)
    h_off, h_eid = sub_segments(off64, hubs_d)
    h_idx64 = u32_to_i64(idx_dev[h_eid])
    h_w = w_dev[h_eid]
    exact = exact_rows_f64(x, h_idx64, h_w, h_off)
    got_h = out[hubs_d].cpu().numpy()
    h_idx, h_wh = host_u32(idx_dev[h_eid]), h_w.cpu().numpy()
    ref_h = oracle.spmm(xh, h_wh, h_off, h_idx, hubs.size)
    scale_h = oracle.spmm(np.abs(xh), h_wh, h_off, h_idx, hubs.size)
    err_gpu, err_cpu = rel_err(got_h, exact, scale_h), rel_err(ref_h, exact, scale_h)
    print(f"{tag}: {int(whole.sum())} uncut rows bit-exact, {rows.size} rows within {err:.2e}; hubs "
          f"{np.diff(h_off.astype(np.int64)).tolist()} vs fp64: gpu {err_gpu:.2e}, sequential oracle {err_cpu:.2e}",
          flush=True)
    assert err_gpu <= TOL and err_gpu <= max(err_cpu, 1e-5), f"{tag}: hub rows"
    return deg


def test_config3_benchmarked_schedule_against_the_oracle(device):
    V, E, chunk_edges, slabs = 232_965, 114_800_000, 512, 32
    src, dst = synth.rmat_edges(V, E, 0.57, 0.19, 0.19, seed=3, device=device, sort=True)
    chunk = FullGraphChunk.from_edges(src, dst, V, chunk_edges, slabs)
    del src, dst
    info = chunk.plan_forward.info()
    assert info["split_rows"] > 10_000 and info["partials"] > 500_000  # the cache-aware schedule is in use
    op = ForwardSingleGPUfuseOp(chunk)
    rows = synth.permutation(V, 7, device)[:3000].cpu().numpy()
    for F, seed in ((602, 31), (128, 32)):
        x = synth.normal_features(V, F, seed=seed, device=device)
        xh = x.cpu().numpy()
        for tag, run, off, idx, w in (
                ("forward", op.forward, chunk.column_offset_gpu, chunk.row_indices_gpu, chunk.edge_weight_forward_gpu),
                ("backward", op.backward, chunk.row_offset_gpu, chunk.column_indices_gpu,
                 chunk.edge_weight_backward_gpu)):
            print(f"case F={F} {tag}", flush=True)
            out = run(x)
            deg_all = u32_to_i64(off)[1:] - u32_to_i64(off)[:-1]
            hubs = torch.topk(deg_all, 6).indices.cpu().numpy()
            deg = check_aggregation_rows(f"F={F} {tag}", out, x, xh, off, idx, w, rows, hubs, chunk_edges // 4)
            # every schedule class is represented in the sample
            assert (deg <= 128).sum() > 300 and ((deg > 128) & (deg <= 512)).sum() > 100 and (deg > 512).sum() > 100
            assert torch.equal(out, run(x))  # bit-reproducible
            del out
        del x, xh


def _oracle_layers(layers, fanouts, gco_h, gri_h, batch_ids, V):
    """Every array of every layer against the restated host algorithms, on the neighbour lists the
    builder picked.  Returns per layer (co, local ri, ro, ci, ewf, ewb, source, destination)."""
    built = []
    dst = batch_ids
    for hop, layer in enumerate(layers[::-1]):
        co = host_u32(layer.dev_column_offset)
        assert np.array_equal(co, oracle.init_co(gco_h, dst, fanouts[hop])), f"hop {hop} init_co"
        local, source = host_u32(layer.dev_row_indices), host_u32(layer.dev_source)
        assert np.array_equal(host_u32(layer.dev_destination), dst)
        glob = source[local]
        for i in range(0, dst.size, 211):  # sampled sources are distinct in-neighbours of their destination
            seg = gri_h[gco_h[dst[i]]:gco_h[dst[i] + 1]]
            mine = glob[co[i]:co[i + 1]]
            assert np.isin(mine, seg).all()
            if fanouts[hop] >= 0 and seg.size > fanouts[hop]:
                assert mine.size == fanouts[hop]
        want_local, want_source, n = oracle.postprocess(glob, V)
        assert n == layer.src_size and np.array_equal(source, want_source) and np.array_equal(local, want_local)
        ro, ci = oracle.csr_from_csc(co, local, n)
        assert np.array_equal(host_u32(layer.dev_row_offset), ro)
        assert np.array_equal(host_u32(layer.dev_column_indices), ci)
        outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
        ewf, ewb = oracle.layer_weights(co, local, ro, ci, source, dst, outd, ind)
        assert layer.dev_ewf().cpu().numpy().tobytes() == ewf.tobytes()
        assert layer.dev_ewb().cpu().numpy().tobytes() == ewb.tobytes()
        built.append(dict(co=co, ri=local, ro=ro, ci=ci, ewf=ewf, ewb=ewb, source=source, destination=dst))
        dst = source
    return built[::-1]


@pytest.fixture(scope="module")
def products_graph(device):
    """The Products-shaped graph of configs 4 and 5: 2,449,029 vertices, 126.2 M R-MAT edges, CSC in
    HBM (uint32 bit patterns) plus host copies for the oracle."""
    cfg = CONFIGS["products"]
    V, E = cfg["V"], cfg["E"]
    assert (V, E) == (2_449_029, 126_200_000)
    src, dst = synth.rmat_edges(V, E, seed=cfg["seed"], device=device, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    out_deg = torch.bincount(src, minlength=V).cpu()
    del src, dst
    gco, gri = as_u32(co), as_u32(ri)
    del co, ri
    return dict(V=V, E=E, gco=gco, gri=gri, out_deg=out_deg, gco_h=host_u32(gco), gri_h=host_u32(gri))


def test_config4_products_full_size_batch(device, products_graph):
    """One batch of 6,000 vertices, fanout [15,10,5], on the whole graph: layers bit-exact, the cached
    gather (489,805 rows in HBM, the rest zero-copy from the 2,449,029 x 100 pinned table) bit-exact
    with the host split's hit count, labels bit-exact, aggregation of the three layers (100, 128, 128
    wide) forward and backward within 1e-4."""
    g = products_graph
    cfg = CONFIGS["products"]
    V, F = g["V"], cfg["F"]
    fanouts = cfg["fanout"]
    assert fanouts == [15, 10, 5] and cfg["batch"] == 6000
    feat_t = synth.normal_features(V, F, seed=cfg["seed"] + 40)
    feat = feat_t.numpy()
    n_cache = int(V * cfg["cache"])
    assert n_cache == 489_805
    table = MappedHostTable(feat_t)
    cache = FeatureCache(feat_t, g["out_deg"], n_cache, device)
    labels = synth.uniform_labels(V, cfg["classes"], seed=cfg["seed"] + 41)
    ids64 = synth.permutation(V, cfg["seed"] + 42, device)[:cfg["batch"]]
    ids = as_u32(ids64)
    builder = BatchBuilder(g["gco"], g["gri"], fanouts, cfg["batch"])
    layers = builder.sample(ids, 4000)
    sizes = [(l.v_size, l.e_size, l.src_size) for l in layers]
    print(f"layers (input side first): {sizes}", flush=True)
    assert layers[-1].v_size == 6000 and layers[0].e_size > 500_000
    built = _oracle_layers(layers, fanouts, g["gco_h"], g["gri_h"], host_u32(ids), V)
    cs = CudaStream()
    # cached gather
    src0 = built[0]["source"]
    want = oracle.get_feature(feat, src0)
    hashmap_ref = oracle.mark_cache(V, cache.order.numpy().astype(np.uint32), n_cache)
    assert np.array_equal(host_u32(cache.dev_cache_node_hashmap), hashmap_ref)
    _, hit, miss = oracle.load_feature_cached(feat, cache.dev_cache_feature.cpu().numpy(), src0, hashmap_ref)
    x0 = torch.full((src0.size, F), float("nan"), device=device)
    hits = load_feature_gpu_cache(cs, layers[0], x0, table.dev_ptr, cache)
    cs.CUDA_DEVICE_SYNCHRONIZE()
    assert x0.cpu().numpy().tobytes() == want.tobytes() and int(hits.item()) == hit.size
    assert hit.size + miss.size == src0.size and hit.size > 0.5 * src0.size
    print(f"gathered {src0.size} rows, {hit.size} from the cache", flush=True)
    # labels of the batch
    lab = torch.empty(layers[-1].v_size, dtype=torch.int64, device=device)
    load_label_gpu(cs, layers[-1], lab, labels.to(device))
    assert np.array_equal(lab.cpu().numpy(), oracle.get_label(labels.numpy(), built[-1]["destination"]))
    # aggregation
    x = x0
    for l, (layer, h) in enumerate(zip(layers, built)):
        print(f"layer {l}: Vd={layer.v_size} E={layer.e_size} Vs={layer.src_size} F={x.shape[1]}", flush=True)
        op = SingleGPUSampleGraphOp(layers, l, cs)
        y = op.forward(x)
        xh = x.cpu().numpy()
        check(y.cpu().numpy(), oracle.spmm(xh, h["ewf"], h["co"], h["ri"], layer.v_size),
              oracle.spmm(np.abs(xh), h["ewf"], h["co"], h["ri"], layer.v_size))
        gy = synth.normal_features(layer.v_size, x.shape[1], seed=50 + l, device=device)
        gx = op.backward(gy)
        gyh = gy.cpu().numpy()
        check(gx.cpu().numpy(), oracle.spmm(gyh, h["ewb"], h["ro"], h["ci"], layer.src_size),
              oracle.spmm(np.abs(gyh), h["ewb"], h["ro"], h["ci"], layer.src_size))
        x = synth.normal_features(layer.v_size, cfg["hidden"], seed=60 + l, device=device)  # the dense layer's output
    builder.close()
    table.close()


def _gat_layer_oracle(co, ri, Vs, hs, el, er, gout, H, Fh):
    """The chain of the reference's CPU operators, head by head (toolkits/GAT_CPU.hpp:178-204):
    scatter -> leaky_relu(0.2) -> SingleEdgeSoftMax -> weighted SingleCPUDstAggregateOp, and back."""
    E, Vd = ri.size, co.size - 1
    pre = (oracle.scatter_src(el, co, ri) + oracle.scatter_dst(er, co, E)).astype(np.float32)
    m = np.where(pre > 0, pre, np.float32(0.2) * pre).astype(np.float32)
    alpha = oracle.edge_softmax(m, co)
    g_eout = oracle.scatter_dst(gout, co, E)
    msg = oracle.scatter_src(hs, co, ri)
    out = np.zeros((Vd, H * Fh), np.float32)
    gal = np.zeros((E, H), np.float32)
    ghs = np.zeros((Vs, H * Fh), np.float32)
    for h in range(H):
        sl = slice(h * Fh, (h + 1) * Fh)
        out[:, sl] = oracle.aggregate_dst(np.ascontiguousarray(msg[:, sl] * alpha[:, h:h + 1]), co)
        gal[:, h] = (g_eout[:, sl].astype(np.float64) * msg[:, sl]).sum(1)
        ghs[:, sl] = oracle.gather_to_src(np.ascontiguousarray(g_eout[:, sl] * alpha[:, h:h + 1]), co, ri, Vs)
    gm = oracle.edge_softmax_bwd(gal, alpha, co)
    gs = (gm * np.where(pre > 0, np.float32(1.0), np.float32(0.2))).astype(np.float32)
    a_exp = np.repeat(alpha, Fh, axis=1)
    scale_gs = alpha * (np.abs(gal) + oracle.scatter_dst(oracle.aggregate_dst(np.abs(gal) * alpha, co), co, E))
    return dict(alpha=alpha, out=out, gal=gal, ghs=ghs, gs=gs, ger=oracle.aggregate_dst(gs, co),
                gel=oracle.gather_to_src(gs, co, ri, Vs),
                scale_out=oracle.aggregate_dst(np.abs(msg) * a_exp, co),
                scale_ghs=oracle.gather_to_src(np.abs(g_eout) * a_exp, co, ri, Vs),
                scale_gal=np.stack([(np.abs(g_eout[:, h * Fh:(h + 1) * Fh]) * np.abs(msg[:, h * Fh:(h + 1) * Fh])).sum(1)
                                    for h in range(H)], 1),
                scale_gs=scale_gs, scale_ger=oracle.aggregate_dst(scale_gs.astype(np.float32), co),
                scale_gel=oracle.gather_to_src(scale_gs.astype(np.float32), co, ri, Vs))


def test_config5_gat_full_size_batch(device, products_graph):
    """One batch of 4,096 vertices, fanout [10,10], on the whole graph: fused attention and the
    attention-weighted aggregation, forward and backward, against the reference's CPU operator chain."""
    g = products_graph
    cfg = CONFIGS["gat"]
    V, H = g["V"], cfg["heads"]
    Fh = cfg["hidden"] // H
    F = H * Fh
    assert cfg["fanout"] == [10, 10] and cfg["batch"] == 4096 and (H, Fh) == (4, 32)
    ids = as_u32(synth.permutation(V, cfg["seed"] + 42, device)[:cfg["batch"]])
    builder = BatchBuilder(g["gco"], g["gri"], cfg["fanout"], cfg["batch"], want_perm=True)
    layers = builder.sample(ids, 5000)
    built = _oracle_layers(layers, cfg["fanout"], g["gco_h"], g["gri_h"], host_u32(ids), V)
    for l, (layer, h) in enumerate(zip(layers, built)):
        Vs, Vd, E = layer.src_size, layer.v_size, layer.e_size
        print(f"layer {l}: Vd={Vd} E={E} Vs={Vs}", flush=True)
        perm = host_u32(layer.dev_csr_to_csc)
        order = np.argsort(h["ri"].astype(np.int64), kind="stable")
        assert np.array_equal(perm, order.astype(np.uint32))
        hs = synth.normal_features(Vs, F, seed=70 + l, device=device)
        hd = synth.normal_features(Vd, F, seed=75 + l, device=device)
        a_l = synth.normal_features(H, Fh, seed=80 + l, device=device) * 0.3
        a_r = synth.normal_features(H, Fh, seed=90 + l, device=device) * 0.3
        gout = synth.normal_features(Vd, F, seed=100 + l, device=device)
        el = torch.einsum("vhf,hf->vh", hs.view(Vs, H, Fh), a_l).contiguous()
        er = torch.einsum("vhf,hf->vh", hd.view(Vd, H, Fh), a_r).contiguous()
        ref = _gat_layer_oracle(h["co"], h["ri"], Vs, hs.cpu().numpy(), el.cpu().numpy(), er.cpu().numpy(),
                                gout.cpu().numpy(), H, Fh)
        att, agg = GATAttentionOp(layer, 0.2), GATAggregateOp(layer, H)
        alpha = att.forward(el, er)
        check(alpha.cpu().numpy(), ref["alpha"], scale=1.0, floor=1e-6)
        # the later stages are fed the oracle's alpha / galpha so that each is checked on equal inputs
        alpha_ref = torch.from_numpy(ref["alpha"]).to(device)
        att.alpha = alpha_ref
        out = agg.forward(hs, alpha_ref)
        check(out.cpu().numpy(), ref["out"], scale=ref["scale_out"])
        ghs = agg.backward(gout)
        check(ghs.cpu().numpy(), ref["ghs"], scale=ref["scale_ghs"])
        check(agg.get_additional_grad().cpu().numpy(), ref["gal"], scale=ref["scale_gal"])
        gel = att.backward(torch.from_numpy(ref["gal"]).to(device))
        check(att.get_additional_grad().cpu().numpy(), ref["ger"], scale=ref["scale_ger"])
        check(gel.cpu().numpy(), ref["gel"], scale=ref["scale_gel"])
    builder.close()


def _seg_reduce(ufunc, v, sub_off):
    return ufunc.reduceat(v, sub_off[:-1].astype(np.int64), axis=0)


def _softmax64(x, sub_off):
    """Per-segment softmax in float64 (no empty segments)."""
    lens = np.diff(sub_off.astype(np.int64))
    x = x.astype(np.float64)
    ex = np.exp(x - np.repeat(_seg_reduce(np.maximum, x, sub_off), lens, axis=0))
    return ex / np.repeat(_seg_reduce(np.add, ex, sub_off), lens, axis=0)


def _softmax_bwd64(gy, y, sub_off):
    lens = np.diff(sub_off.astype(np.int64))
    gy, y = gy.astype(np.float64), y.astype(np.float64)
    return y * (gy - np.repeat(_seg_reduce(np.add, gy * y, sub_off), lens, axis=0))


def _check_segments(tag, got, ref, exact, short, scale, floor=1e-2):
    """Segments of at most 32,768 edges (`short`, per edge): directly against the oracle.  Longer ones
    are summed in pieces on the GPU and strictly sequentially by the oracle, two fp32 orders that
    differ by ~sqrt(n) ulp legitimately: both are measured against float64, the GPU has to meet the
    tolerance and must not be less accurate than the oracle."""
    sc = scale if np.isscalar(scale) else scale[short]
    check(got[short], ref[short], scale=sc, floor=floor)
    long_ = ~short
    scl = scale if np.isscalar(scale) else scale[long_]
    err_gpu = rel_err(got[long_], exact[long_], scl, floor)
    err_cpu = rel_err(ref[long_], exact[long_], scl, floor)
    print(f"{tag}: {int(long_.sum())} values in long segments vs float64: gpu {err_gpu:.2e}, sequential oracle "
          f"{err_cpu:.2e}", flush=True)
    assert err_gpu <= TOL and err_gpu <= max(err_cpu, 1e-5), tag
    err_all = rel_err(got, exact, scale, floor)
    assert err_all <= TOL, f"{tag}: against float64 {err_all:.3e}"


def test_config5_full_graph_softmax_and_attention_segments(device, products_graph):
    """nts_edge_softmax_fwd/bwd and nts_gat_attention_fwd/bwd over all 126.2 M edges (H = 4); 2,000
    seeded destination segments and the eight longest (the longest has ~3e5 edges: the `pieces` class)
    are compared with the oracle."""
    g = products_graph
    V, E, H = g["V"], g["E"], 4
    gco, gri = g["gco"], g["gri"]
    s = stream()
    off64 = u32_to_i64(gco)
    deg = off64[1:] - off64[:-1]
    hubs = torch.topk(deg, 8).indices
    assert int(deg.max()) > 250_000
    cand = synth.permutation(V, 9, device)
    rows = torch.cat([cand[deg[cand] > 0][:2000], hubs])
    sub_off, eid = sub_segments(off64, rows)
    lens = np.diff(sub_off.astype(np.int64))
    short = np.repeat(lens <= 32768, lens)
    print(f"segments: {rows.numel()} rows, {eid.numel()} edges, longest {int(deg.max())}, "
          f"{int((lens > 32768).sum())} above 32,768 edges", flush=True)

    def seg_sum(v):  # per-row sums over the sub-CSC, broadcast back to its edges
        return np.repeat(_seg_reduce(np.add, v.astype(np.float64), sub_off), lens, axis=0)

    # plain edge softmax
    x = synth.normal_features(E, H, seed=201, device=device) * 3.0
    y = torch.empty_like(x)
    call("nts_edge_softmax_fwd", ptr(y), ptr(x), ptr(gco), V, H, s)
    x_sub = x[eid].cpu().numpy()
    _check_segments("softmax fwd", y[eid].cpu().numpy(), oracle.edge_softmax(x_sub, sub_off), _softmax64(x_sub, sub_off),
                    short, 1.0, floor=1e-6)
    gy = synth.normal_features(E, H, seed=202, device=device)
    gx = torch.empty_like(x)
    call("nts_edge_softmax_bwd", ptr(gx), ptr(gy), ptr(y), ptr(gco), V, H, s)
    y_sub, gy_sub = y[eid].cpu().numpy(), gy[eid].cpu().numpy()
    # on the library's own y: the backward alone
    _check_segments("softmax bwd", gx[eid].cpu().numpy(), oracle.edge_softmax_bwd(gy_sub, y_sub, sub_off),
                    _softmax_bwd64(gy_sub, y_sub, sub_off), short,
                    y_sub * (np.abs(gy_sub) + seg_sum(np.abs(gy_sub) * y_sub)))
    del x, gx
    # fused attention
    el = synth.normal_features(V, H, seed=203, device=device)
    er = synth.normal_features(V, H, seed=204, device=device)
    alpha = torch.empty(E, H, device=device)
    call("nts_gat_attention_fwd", ptr(alpha), ptr(el), ptr(er), ptr(gco), ptr(gri), V, H, 0.2, s)
    src_sub = u32_to_i64(gri[eid])
    dst_sub = torch.repeat_interleave(rows, torch.from_numpy(lens).to(device))
    pre = (el[src_sub] + er[dst_sub]).cpu().numpy()  # fp32 add of two fp32 values: one rounding, as on the CPU
    m = np.where(pre > 0, pre, np.float32(0.2) * pre).astype(np.float32)
    a_sub = alpha[eid].cpu().numpy()
    _check_segments("attention fwd", a_sub, oracle.edge_softmax(m, sub_off), _softmax64(m, sub_off), short, 1.0,
                    floor=1e-6)
    gs = torch.empty(E, H, device=device)
    ger = torch.empty(V, H, device=device)
    call("nts_gat_attention_bwd", ptr(gs), ptr(ger), ptr(gy), ptr(alpha), ptr(el), ptr(er), ptr(gco), ptr(gri), V, H,
         0.2, s)
    slope = np.where(pre > 0, 1.0, 0.2)
    gs_ref = (oracle.edge_softmax_bwd(gy_sub, a_sub, sub_off) * slope.astype(np.float32)).astype(np.float32)
    gs_exact = _softmax_bwd64(gy_sub, a_sub, sub_off) * slope
    scale_gs = a_sub * (np.abs(gy_sub) + seg_sum(np.abs(gy_sub) * a_sub))
    _check_segments("attention bwd (edge scores)", gs[eid].cpu().numpy(), gs_ref, gs_exact, short, scale_gs)
    short_rows = lens <= 32768
    _check_segments("attention bwd (destinations)", ger[rows].cpu().numpy(), oracle.aggregate_dst(gs_ref, sub_off),
                    _seg_reduce(np.add, gs_exact, sub_off), np.repeat(short_rows[:, None], H, 1),
                    _seg_reduce(np.add, scale_gs.astype(np.float64), sub_off))


@pytest.mark.parametrize("F", [4, 32])
def test_config5_full_graph_edge_sums_to_destinations(device, products_graph, F):
    """nts_gather_edge_to_dst over all 126.2 M edges (F = 4: a value per head; F = 32): wavefronts stream
    the contiguous edges of their rows, the first blocks of the launch take the rows above 1,024 edges
    and the pieces of the giant ones.  2,000 seeded destinations and the eight longest against the
    float64 sum (1e-4 of the sum of magnitudes); rows of at most 1,024 edges equal the running fp32
    sum in edge order bit for bit; untouched rows of an accumulating call keep their contents."""
    g = products_graph
    V, E = g["V"], g["E"]
    gco = g["gco"]
    s = stream()
    off64 = u32_to_i64(gco)
    deg = off64[1:] - off64[:-1]
    hubs = torch.topk(deg, 8).indices
    cand = synth.permutation(V, 19, device)
    rows = torch.cat([cand[:2000], hubs])
    sub_off, eid = sub_segments(off64, rows)
    lens = np.diff(sub_off.astype(np.int64))
    print(f"F={F}: {rows.numel()} rows, {eid.numel()} edges, longest {int(deg.max())}, empty {int((lens == 0).sum())}",
          flush=True)
    msg = synth.normal_features(E, F, seed=230 + F, device=device)
    out = torch.full((V, F), float("nan"), device=device)
    call("nts_gather_edge_to_dst", ptr(out), ptr(msg), ptr(gco), V, F, 0, s)
    got = out[rows].cpu().numpy()
    m = msg[eid].cpu().numpy()
    exact = np.zeros((rows.numel(), F))
    scale = np.zeros((rows.numel(), F))
    chain = np.zeros((rows.numel(), F), np.float32)
    for k in range(rows.numel()):
        seg = m[sub_off[k]:sub_off[k + 1]]
        exact[k] = seg.astype(np.float64).sum(0)
        scale[k] = np.abs(seg).astype(np.float64).sum(0)
        if 0 < lens[k] <= 1024:
            chain[k] = np.cumsum(seg, axis=0, dtype=np.float32)[-1]
    assert np.all(np.abs(got - exact) <= 1e-4 * np.maximum(scale, 1e-6)), "beyond 1e-4 of the sum of magnitudes"
    ordered = lens <= 1024
    assert np.array_equal(got[ordered].view(np.uint32), chain[ordered].view(np.uint32))
    assert bool((out == out).all()), "a row was not written"
    # accumulate: out += sums; a second pass doubles nothing but adds once more
    call("nts_gather_edge_to_dst", ptr(out), ptr(msg), ptr(gco), V, F, 1, s)
    twice = out[rows].cpu().numpy()
    assert np.array_equal(twice[ordered], (chain + chain)[ordered])
