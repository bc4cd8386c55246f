"""Per-operator timings of the edge, attention, gather and layout entry points at the Products-shaped
scale (2,449,029 vertices, 126.2 M R-MAT edges), each next to its algorithmic bytes.

    python -m neutronbench_amd.opbench [--scale S] [--reps N]

One JSON line per operator: milliseconds per call (HIP events around `reps` back-to-back calls after
two warm-ups), algorithmic bytes (edge-gather model: every edge reads what it needs once, every
output is written once) and the rate they imply, with its fraction of the 8 TB/s HBM peak.  Rates
above the peak mean re-use out of the caches.  Score / softmax operators run on the whole graph with
4 heads; the operators that move [E, F'] edge messages run on the edges of the first 400,000
destinations (an [E, 32] tensor of the whole graph would be 16 GB per operand); the PCIe rows come
from mapped pinned host memory.
"""
import argparse
import json

import torch

from . import synth
from .abi import call, ptr
from .batch import MappedHostTable
from .layout import SpmmPlan, as_u32

HBM_PEAK = 8.0e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--reps", type=int, default=5)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    V, E = int(2_449_029 * args.scale), int(126_200_000 * args.scale)
    src, dst = synth.rmat_edges(V, E, seed=4, device=dev, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    del src, dst
    co32, ri32 = as_u32(co), as_u32(ri)
    s = torch.cuda.current_stream().cuda_stream

    def report(op, fn, nbytes, note=""):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / args.reps
        rate = nbytes / (ms * 1e-3)
        print(json.dumps({"op": op, "ms": round(ms, 4), "algorithmic_bytes": int(nbytes),
                          "GB_per_s": round(rate / 1e9, 1), "frac_of_hbm_peak": round(rate / HBM_PEAK, 4),
                          "note": note}), flush=True)

    H, Fh = 4, 32
    F = H * Fh
    x = torch.randn(E, H, device=dev)
    y = torch.empty_like(x)
    g = torch.randn(E, H, device=dev)
    gx = torch.empty_like(x)
    whole = f"whole graph, E={E}, H={H}"
    report("nts_edge_softmax_fwd", lambda: call("nts_edge_softmax_fwd", ptr(y), ptr(x), ptr(co32), V, H, s),
           8 * E * H + 4 * (V + 1), whole)
    report("nts_edge_softmax_bwd", lambda: call("nts_edge_softmax_bwd", ptr(gx), ptr(g), ptr(y), ptr(co32), V, H, s),
           12 * E * H + 4 * (V + 1), whole)
    el, er = torch.randn(V, H, device=dev), torch.randn(V, H, device=dev)
    ger = torch.empty(V, H, device=dev)
    report("nts_gat_attention_fwd",
           lambda: call("nts_gat_attention_fwd", ptr(y), ptr(el), ptr(er), ptr(co32), ptr(ri32), V, H, 0.2, s),
           E * (4 + 4 * H + 4 * H) + V * H * 4 + 4 * (V + 1), whole)
    report("nts_gat_attention_bwd",
           lambda: call("nts_gat_attention_bwd", ptr(gx), ptr(ger), ptr(g), ptr(y), ptr(el), ptr(er), ptr(co32),
                        ptr(ri32), V, H, 0.2, s),
           E * (4 + 4 * H * 4) + V * H * 8 + 4 * (V + 1), whole + "; writes the per-edge gradient and the destination-side sum")
    h = torch.randn(V, F, device=dev)
    out = torch.empty_like(h)
    heads_bytes = E * (4 * F + 4 + 4 * H) + V * 4 * F + 4 * (V + 1)
    report("nts_spmm_gather_heads", lambda: call("nts_spmm_gather_heads", ptr(h), ptr(out), ptr(y), 0, ptr(co32),
                                                  ptr(ri32), V, E, H, Fh, 0, s), heads_bytes,
           whole + f", F'={F}, no plan: hub rows cut on the device")
    plan = SpmmPlan(co32, V, E, 512, indices=ri32, n_index=V, n_slabs=32)
    plan.reserve(F)
    report("nts_spmm_gather_heads_planned",
           lambda: call("nts_spmm_gather_heads_planned", plan.handle, ptr(h), ptr(out), ptr(y), 0, ptr(co32), ptr(ri32),
                        H, Fh, 0, s), heads_bytes, whole + f", F'={F}, pieces <= 512 edges, 32 source ranges")
    w = torch.rand(E, device=dev)
    report("nts_spmm_gather (no plan)", lambda: call("nts_spmm_gather", ptr(h), ptr(out), ptr(w), ptr(co32), ptr(ri32),
                                                      0, V, E, F, 0, s),
           E * (4 * F + 8) + V * 4 * F + 4 * (V + 1), whole + f", F={F}, hub rows cut on the device")
    report("nts_spmm_gather_planned", lambda: call("nts_spmm_gather_planned", plan.handle, ptr(h), ptr(out), ptr(w),
                                                    ptr(co32), ptr(ri32), 0, F, 0, s),
           E * (4 * F + 8) + V * 4 * F + 4 * (V + 1), whole + f", F={F}")
    report("nts_sddmm_heads", lambda: call("nts_sddmm_heads", ptr(gx), ptr(h), ptr(out), ptr(co32), ptr(ri32), V, H, Fh,
                                            s), E * (4 * F + 4 + 4 * H) + V * 4 * F, whole + f", F'={F}")
    plan.close()
    del x, y, g, gx, h, out, w

    Vd = min(V, int(400_000 * args.scale))
    E2 = int(co[Vd])
    Fm = 32
    msg = torch.empty(E2, Fm, device=dev)
    feat = torch.randn(V, Fm, device=dev)
    o_dst = torch.empty(Vd, Fm, device=dev)
    part = f"edges of the first {Vd} destinations, E={E2}, F'={Fm}"
    report("nts_scatter_src_to_edge", lambda: call("nts_scatter_src_to_edge", ptr(msg), ptr(feat), ptr(ri32), ptr(co32), 0,
                                                    Vd, Fm, s), E2 * (8 * Fm + 4), part)
    report("nts_scatter_dst_to_edge", lambda: call("nts_scatter_dst_to_edge", ptr(msg), ptr(feat), ptr(co32), Vd, Fm, s),
           E2 * 4 * Fm + Vd * 4 * Fm, part)
    report("nts_gather_edge_to_dst", lambda: call("nts_gather_edge_to_dst", ptr(o_dst), ptr(msg), ptr(co32), Vd, Fm, 0, s),
           E2 * 4 * Fm + Vd * 4 * Fm, part)
    del msg, feat, o_dst
    Fw = 128  # edge rows as wide as a hidden layer: what the unfused GAT aggregation sums
    msg = torch.randn(E2, Fw, device=dev)
    o_dst = torch.empty(Vd, Fw, device=dev)
    report("nts_gather_edge_to_dst (wide rows)", lambda: call("nts_gather_edge_to_dst", ptr(o_dst), ptr(msg), ptr(co32), Vd,
                                                              Fw, 0, s),
           E2 * 4 * Fw + Vd * 4 * Fw, f"edges of the first {Vd} destinations, E={E2}, F'={Fw}")
    del msg, o_dst

    n = int(1_000_000 * args.scale)
    Ff = 100
    table_dev = torch.randn(V, Ff, device=dev)
    ids = as_u32((synth.hash64(torch.arange(n, device=dev), 5) & 0x7FFFFFFF) % V)
    o = torch.empty(n, Ff, device=dev)
    report("nts_gather_rows_f32 (HBM table)", lambda: call("nts_gather_rows_f32", ptr(o), ptr(table_dev), ptr(ids), 0, 0,
                                                            n, Ff, s), n * (8 * Ff + 4), f"{n} random rows of {Ff} floats")
    labels = torch.randint(0, 47, (V,), device=dev)
    lo = torch.empty(n, dtype=torch.int64, device=dev)
    report("nts_gather_labels_i64", lambda: call("nts_gather_labels_i64", ptr(lo), ptr(labels), ptr(ids), n, 1, s),
           n * 20, f"{n} labels")
    host = MappedHostTable(table_dev.cpu())
    report("nts_gather_rows_f32 (mapped pinned host)", lambda: call("nts_gather_rows_f32", ptr(o), host.dev_ptr, ptr(ids),
                                                                    0, 0, n, Ff, s), n * 4 * Ff,
           f"{n} random rows of {Ff} floats over PCIe; bytes = PCIe payload (ceiling measured with hipMemcpy: ~57 GB/s)")
    n_cache = V // 5
    order = torch.argsort(synth.hash64(torch.arange(V, device=dev), 9))[:n_cache]
    hashmap = torch.full((V,), -1, dtype=torch.int32, device=dev)
    hashmap[order] = torch.arange(n_cache, dtype=torch.int32, device=dev)
    cache = table_dev[order].contiguous()
    hits = torch.zeros(1, dtype=torch.int32, device=dev)
    miss = int((hashmap[ids.to(torch.int64) & 0xFFFFFFFF] < 0).sum())
    report("nts_gather_rows_cached_f32", lambda: call("nts_gather_rows_cached_f32", ptr(o), host.dev_ptr, ptr(cache),
                                                       ptr(ids), ptr(hashmap), n, Ff, ptr(hits), s), miss * 4 * Ff,
           f"{n} rows, {n - miss} from the HBM cache, {miss} over PCIe; bytes = PCIe payload")
    host.close()


if __name__ == "__main__":
    main()
