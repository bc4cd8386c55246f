#!/usr/bin/env python3
"""Benchmark of the aggregation hot path on one MI355X.

Workload (BASELINE.json configs[2]): Reddit-shaped full-graph 2-layer GCN aggregation,
forward + backward, whole graph resident in HBM.  232,965 vertices, 114.8 M directed R-MAT edges,
GCN-normalised edge weights, fp32.  One step = the four aggregations of one training iteration in
aggregate-then-transform order: layer-0 forward (F=602), layer-1 forward (F=128), layer-1 backward
(F=128), layer-0 backward (F=602).  Forward gathers by destination over the CSC, backward gathers
by source over the CSR.  Inputs are resident in HBM before the timed region.

Prints one JSON line: edges aggregated per second (4 * E edges per step); the roofline figure of the
dominant kernel (the F=602 gather): its HBM-side bytes per launch from the committed rocprofv3
counter summary over the kernel time this run measures with HIP events recorded around that kernel;
a check of the last timed step's outputs against the CPU oracle; and the CPU baselines timed on the
host cores on the same graph: the reference's own CPU operator where the reference-built program
oracle/_ref/ref_fullgraph_cpu is present ("reference"), and the CPU oracle ("port") at both thread
settings.  The run exits with status 1 when the check fails.

--workload arxiv|products|gat measures the per-epoch time of that sampled mini-batch configuration
instead (sampling, layer construction, gathers, aggregation fwd+bwd, all through the C ABI) and
prints it in the same format, with the CPU oracle timed on a few batches of the same epoch.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

V_REDDIT = 232_965
E_REDDIT = 114_800_000
F_IN, F_HID = 602, 128
# The reference's own operators, built from the reference tree where that is present (test infrastructure):
# its CPU operator, and its GPU operator class compiled against this library's host veneer.
REFERENCE_PROGRAM = os.path.join(ROOT, "oracle", "_ref", "ref_fullgraph_cpu")
REFERENCE_GPU_PROGRAM = os.path.join(ROOT, "oracle", "_ref", "ref_fullgraph_gpu")
# The reference's own sampler and mini-batch CPU operator behind a small driver (oracle/ref_minibatch_driver.cpp,
# built by oracle/build_toolkits.sh where the reference tree is present).
REFERENCE_MINIBATCH_PROGRAM = os.path.join(ROOT, "oracle", "_ref", "ref_minibatch")
HBM_PEAK_GBS = 8000.0
# rocprofv3 counter summary of the dominant kernel on this workload; it names the kernel sources it was
# measured with, and its traffic figure is only quoted while those sources are unchanged.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "spmm_wave_f602_reddit_shaped_pmc.txt")
KERNEL_SOURCES = [os.path.join(ROOT, "neutronbench_amd", "csrc", n) for n in ("spmm.hip", "common.hpp")]


def algorithmic_bytes(E, V_out, F, weighted=True):
    """Edge-gather model of one aggregation pass: one source row, one index and one weight per
    edge; one output row and one offset per output row."""
    return E * (4 * F + 4 + (4 if weighted else 0)) + V_out * 4 * F + (V_out + 1) * 4


def compulsory_bytes(E, V_in, V_out, F):
    """Every input and output row once, every index and weight once, every offset once."""
    return (V_in + V_out) * 4 * F + E * 8 + (V_out + 1) * 4


def kernel_sources_digest():
    import hashlib

    h = hashlib.sha256()
    for path in KERNEL_SOURCES:
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """HBM-side bytes per launch of the dominant kernel from the committed rocprofv3 summary
    (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a plain copy), or None
    when the summary is missing, was taken on another workload / schedule, or with other kernel
    sources than the ones this run uses."""
    try:
        fields = {}
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if ":" in line and not line.startswith(" "):
                    k, v = line.split(":", 1)
                    fields[k.strip()] = v.strip()
        if fields.get("kernel_sources_sha256_16") != kernel_sources_digest():
            return None
        if fields.get("workload") != workload:
            return None
        return {"traffic": int(fields["traffic_bytes_per_launch"]), "fetch": int(fields["fetch_bytes_per_launch"]),
                "write": int(fields["write_bytes_per_launch"]), "kernel": fields.get("kernel"),
                "l2_hit_rate": float(fields["l2_hit_rate"]) if "l2_hit_rate" in fields else None,
                "l2_request_bytes": int(fields["l2_request_bytes_per_launch"]) if "l2_request_bytes_per_launch" in fields else None}
    except (OSError, KeyError, ValueError):
        return None


def reddit_graph(torch, V, E, distinct, chunk, slabs, dev):
    """The Reddit-shaped chunk: R-MAT a=.57 b=.19 c=.19, seed 3, ids permuted, edge list in (src, dst)
    order.  distinct=True: the first E distinct pairs of the draw sequence (a simple graph, as the Reddit
    graph itself is); False: the first E draws, parallel edges kept."""
    from neutronbench_amd import synth
    from neutronbench_amd.layout import FullGraphChunk

    src, dst = synth.rmat_edges(V, E, 0.57, 0.19, 0.19, seed=3, device=dev, sort=True, distinct=distinct)
    chunk_obj = FullGraphChunk.from_edges(src, dst, V, chunk, slabs)
    del src, dst
    return chunk_obj


def time_steps(torch, chunk, tensors, steps, warmup):
    """`warmup` untimed and `steps` timed steps (fwd F=602, fwd F=128, bwd F=128, bwd F=602) of the
    operator mirror over `chunk`.  Returns (seconds for the timed steps, per-pass gather-kernel ms from
    HIP events recorded by the library around its main kernel, the last step's four outputs)."""
    from neutronbench_amd.abi import call
    from neutronbench_amd.ops import ForwardSingleGPUfuseOp

    x0, h1, g1, g0 = tensors
    op = ForwardSingleGPUfuseOp(chunk, with_weight=True)
    chunk.plan_forward.reserve(F_IN)
    chunk.plan_backward.reserve(F_IN)
    for _ in range(warmup):
        op.forward(x0), op.forward(h1), op.backward(g1), op.backward(g0)
    torch.cuda.synchronize()
    # One HIP event pair per aggregation launch of the timed region (4 per step).  The library records
    # them on the launch stream immediately before and after its main gather kernel; nothing waits on
    # them until the timed region is over.
    events = []
    for _ in range(4 * steps):
        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        call("nts_event_create", ctypes.byref(a))
        call("nts_event_create", ctypes.byref(b))
        events.append((a, b))
    fwd, bwd = chunk.plan_forward.handle, chunk.plan_backward.handle
    outs = [None] * 4

    def timed_step(i):
        call("nts_spmm_plan_set_events", fwd, *events[4 * i + 0])
        outs[0] = op.forward(x0)    # layer 0: aggregate the 602-wide input features
        call("nts_spmm_plan_set_events", fwd, *events[4 * i + 1])
        outs[1] = op.forward(h1)    # layer 1: aggregate the 128-wide hidden features
        call("nts_spmm_plan_set_events", bwd, *events[4 * i + 2])
        outs[2] = op.backward(g1)   # layer 1 backward: gradient gather over the CSR
        call("nts_spmm_plan_set_events", bwd, *events[4 * i + 3])
        outs[3] = op.backward(g0)   # layer 0 backward

    # Timed region: exactly `steps` steps between two synchronisations.
    torch.cuda.synchronize()
    t_start = time.perf_counter()
    for i in range(steps):
        timed_step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_start
    call("nts_spmm_plan_set_events", fwd, None, None)
    call("nts_spmm_plan_set_events", bwd, None, None)
    durs = []
    for a, b in events:
        ms = ctypes.c_float()
        call("nts_event_elapsed_ms", ctypes.byref(ms), a, b)
        durs.append(ms.value)
        call("nts_event_destroy", a)
        call("nts_event_destroy", b)
    per_pass = [sum(durs[k::4]) / steps for k in range(4)]  # fwd602, fwd128, bwd128, bwd602
    # Whole passes (padded copy where there is one, gather, second stage of the cut rows), each timed
    # alone with events on the launch stream, outside the timed region.
    whole = []
    for run, x in ((op.forward, x0), (op.forward, h1), (op.backward, g1), (op.backward, g0)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            run(x)
        e1.record()
        torch.cuda.synchronize()
        whole.append(e0.elapsed_time(e1) / 5)
    return elapsed, per_pass, whole, list(outs)


PASS_NAMES = ("fwd_F602", "fwd_F128", "bwd_F128", "bwd_F602")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--vertices", type=int, default=V_REDDIT)
    ap.add_argument("--edges", type=int, default=E_REDDIT)
    ap.add_argument("--chunk", type=int, default=512, help="largest number of edges in one piece of a split hub row")
    ap.add_argument("--slabs", type=int, default=32,
                    help="source ranges of the cache-aware schedule (1 = split hub rows by edge count only)")
    ap.add_argument("--graph", choices=["simple", "multigraph"], default="simple",
                    help="simple (default): the first E distinct R-MAT pairs, a simple graph like the Reddit graph; "
                         "multigraph: the first E draws with parallel edges kept (timed beside the headline anyway)")
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip everything that runs on the host after the timed region: the check of the timed "
                         "outputs against the CPU oracle, the CPU baselines and the reference operator's time")
    ap.add_argument("--no-epochs", action="store_true",
                    help="skip the three sampled mini-batch epochs (BASELINE.json configs 2, 4, 5) of the default run")
    ap.add_argument("--no-other-graph", action="store_true", help="skip the steps on the other kind of graph")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one plain 1 GiB row copy (identity gather) so that HBM byte counters can be scaled")
    ap.add_argument("--cpu-reps", type=int, default=5, help="timed repetitions of each CPU baseline (median reported)")
    ap.add_argument("--cpu-reference-edges", type=int, default=0,
                    help="edges of the graph the reference's own operators are timed on (0 = the whole graph; a "
                         "smaller number takes the edges of the lowest-numbered source vertices)")
    ap.add_argument("--workload", choices=["reddit", "arxiv", "products", "gat"], default="reddit",
                    help="reddit (default): the aggregation workload above, with the three epochs beside it; arxiv / "
                         "products / gat: only the per-epoch time of that sampled mini-batch configuration")
    ap.add_argument("--cpu-batches", type=int, default=3, help="mini-batch workloads: batches the CPU oracle is timed on")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")
    if args.workload != "reddit":
        return run_epoch_workload(args)

    import torch

    from neutronbench_amd import synth
    from neutronbench_amd.abi import call, ptr

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP library has no CPU fallback)")
    dev = torch.device("cuda:0")
    V, E = args.vertices, args.edges
    simple = args.graph == "simple"

    t0 = time.time()
    chunk = reddit_graph(torch, V, E, simple, args.chunk, args.slabs, dev)
    x0 = synth.normal_features(V, F_IN, seed=31, device=dev)
    h1 = synth.normal_features(V, F_HID, seed=32, device=dev)
    g1 = synth.normal_features(V, F_HID, seed=33, device=dev)
    g0 = synth.normal_features(V, F_IN, seed=34, device=dev)
    tensors = (x0, h1, g1, g0)
    torch.cuda.synchronize()
    setup_s = time.time() - t0
    chunk.plan_forward.reserve(F_IN)
    chunk.plan_backward.reserve(F_IN)
    scratch = [p.scratch_info(F_IN) for p in (chunk.plan_forward, chunk.plan_backward)]

    if args.calibrate:
        # Plain copy of known size: 2^18 rows of 1024 floats = 1 GiB read + 1 GiB written (+ 1 MiB of ids).
        n_cal, f_cal = 1 << 18, 1024
        cal_src = torch.ones(n_cal, f_cal, device=dev)
        cal_dst = torch.empty_like(cal_src)
        cal_ids = torch.arange(n_cal, dtype=torch.int32, device=dev)
        call("nts_gather_rows_f32", ptr(cal_dst), ptr(cal_src), ptr(cal_ids), 0, 0, n_cal, f_cal,
             torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        del cal_src, cal_dst, cal_ids

    elapsed, per_pass, whole, outs = time_steps(torch, chunk, tensors, args.steps, args.warmup)
    ms_per_step = elapsed * 1e3 / args.steps
    edges_per_s = 4.0 * E / (elapsed / args.steps)

    # Dominant kernel: the F=602 gather (spmm_wave_kernel), launched twice per step: forward over the
    # CSC and backward over the CSR.  Same algorithmic bytes per launch for both.
    kernel_ms = (per_pass[0] + per_pass[3]) / 2
    algo = algorithmic_bytes(E, V, F_IN)
    compulsory = compulsory_bytes(E, V, V, F_IN)
    model_gbs = algo / (kernel_ms * 1e-3) / 1e9
    workload_key = f"V={V} E={E} graph={args.graph} chunk={args.chunk} slabs={args.slabs} F={F_IN}"
    measured = measured_traffic(workload_key)
    padded = scratch[0]["padded_input_bytes"] > 0
    fabric_gbs = measured["traffic"] / (kernel_ms * 1e-3) / 1e9 if measured else None
    roofline = {
        # What bounds the kernel: the path behind the L2 -- Infinity Cache and HBM together.  No counter of
        # this GPU tells an Infinity Cache hit from an HBM read, so `traffic` (FETCH_SIZE + WRITE_SIZE of
        # rocprofv3, counted where the L2 talks to the fabric) is an upper bound of the HBM bytes, and
        # `achieved` / `frac` are that traffic over this run's kernel time against the HBM peak.
        "bound": "l2+fabric",
        "kernel": (measured or {}).get("kernel") or
        ("spmm_wave_kernel<4,3,...> over a padded input copy" if padded else "spmm_wave_kernel<1,10,...>")
        + " (F=602 gather, forward and backward launches)",
        "achieved": round(fabric_gbs, 1) if measured else None,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(fabric_gbs / HBM_PEAK_GBS, 4) if measured else None,
        "traffic": measured["traffic"] if measured else None,
        "traffic_source": ("profiles/spmm_wave_f602_reddit_shaped_pmc.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per "
                           "launch of this kernel on this workload, each scaled by the same counter's reading for a "
                           "plain copy; quoted only while the sha256 of the kernel sources recorded there matches the "
                           "sources of this run") if measured else "no counter summary matches this run's kernel sources",
        "l2_request_bytes": (measured or {}).get("l2_request_bytes"),
        "l2_hit_rate": (measured or {}).get("l2_hit_rate"),
        "target_frac": 0.6,
        "target_met": bool(measured and fabric_gbs / HBM_PEAK_GBS >= 0.6),
        "target_basis": "L2-miss traffic (Infinity Cache hits included: an upper bound of the HBM bytes) over the HBM peak",
        # every array once, over the same kernel time: the share of the HBM peak spent on bytes that must move
        "compulsory_bytes": compulsory,
        "compulsory_frac": round(compulsory / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        # the edge-gather model (one source row per edge) counts every re-read served by L2 as a byte
        # moved; it exceeds the HBM peak and is reported for comparison only
        "algorithmic_bytes": algo,
        "model_gbs": round(model_gbs, 1),
        "model_frac": round(model_gbs / HBM_PEAK_GBS, 4),
        "kernel_ms": round(kernel_ms, 3),
        "per_pass_ms": {n: round(v, 3) for n, v in zip(PASS_NAMES, per_pass)},
        # the whole call: padded copy where there is one + gather + second stage of the cut rows
        "pass_ms": {n: round(v, 3) for n, v in zip(PASS_NAMES, whole)},
    }

    check = cpu_baseline = None
    reference_operator = None
    if not args.no_cpu_baseline:
        inputs = dict(zip(PASS_NAMES, tensors))
        check = check_against_oracle(torch, chunk, inputs, dict(zip(PASS_NAMES, outs)), V)
        if not check["ok"]:
            print(json.dumps({"error": "timed outputs differ from the CPU oracle", "check": check}))
            sys.exit(1)
        ref_edges = min(E, args.cpu_reference_edges) if args.cpu_reference_edges > 0 else E
        cpu_baseline, reference_operator = run_reference_programs(torch, chunk, x0, h1, V, ref_edges, args.cpu_reps)
        port = run_cpu_port_baseline(torch, chunk, x0, h1, g1, g0, V, args.cpu_reps)
        if cpu_baseline is None:
            cpu_baseline = port.pop("all_threads")
            cpu_baseline["other_thread_setting"] = port.pop("reference_default_threads")
        else:
            cpu_baseline["port"] = port
    plan_info = dict(chunk.plan_forward.info(), chunk_edges=args.chunk, slabs=args.slabs)
    plan_build_s = chunk.plan_build_s
    del chunk, outs
    torch.cuda.empty_cache()

    # The same step on the other kind of graph, outside the headline: the same R-MAT draws with parallel
    # edges kept (a multigraph: the kernel then loads a source row once per run of equal neighbours).
    other = None
    if not args.no_other_graph:
        chunk2 = reddit_graph(torch, V, E, not simple, args.chunk, args.slabs, dev)
        el2, pp2, whole2, _ = time_steps(torch, chunk2, tensors, max(3, args.steps // 2), 2)
        n2 = max(3, args.steps // 2)
        sc2 = chunk2.plan_forward.scratch_info(F_IN)
        other = {
            "graph": ("the first E R-MAT draws, parallel edges kept" if simple else "the first E distinct R-MAT pairs"),
            "ms_per_step": round(el2 * 1e3 / n2, 3),
            "edges_per_s": round(4.0 * E / (el2 / n2), 1),
            "per_pass_ms": {n: round(v, 3) for n, v in zip(PASS_NAMES, pp2)},
            "pass_ms": {n: round(v, 3) for n, v in zip(PASS_NAMES, whole2)},
            "repeated_edges": sc2["repeated_edges"],
            "loads_once_per_run": sc2["loads_once_per_run"],
            "note": "edges that repeat the neighbour of the edge before them in their row are parallel edges; with "
                    "at least 1 in 20 such edges the kernel loads a row once per run and adds it once per edge, "
                    "which is where a multigraph's higher rate comes from -- it does not apply to a simple graph",
        }
        del chunk2
        torch.cuda.empty_cache()
    del x0, h1, g1, g0, tensors
    torch.cuda.empty_cache()

    epochs = None
    if not args.no_epochs:
        epochs = run_epochs(torch, ("arxiv", "products", "gat"), not args.no_cpu_baseline, args.cpu_batches)
        bad = [n for n, e in epochs.items() if e.get("check") and not e["check"]["ok"]]
        if bad:
            print(json.dumps({"error": f"epoch batch of {bad} differs from the CPU oracle", "epochs": epochs}))
            sys.exit(1)

    out = {
        "metric": "edges aggregated/s (fwd+bwd)",
        "value": round(edges_per_s, 1),
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "Reddit-shaped full-graph 2-layer GCN aggregation fwd+bwd (F=602,128)",
            "vertices": V,
            "edges": E,
            "graph": "R-MAT a=.57 b=.19 c=.19, seed 3, ids permuted, edge list in (src, dst) order; "
                     + ("the first E distinct pairs of the draw sequence: a simple graph, as the Reddit graph is"
                        if simple else "the first E draws, parallel edges kept"),
            "parallel_edges": {"forward": scratch[0]["repeated_edges"], "backward": scratch[1]["repeated_edges"],
                               "loads_once_per_run": scratch[0]["loads_once_per_run"]},
            "other_graph": other,
            "passes_per_step": 4,
            "plan": plan_info,
            "plan_build_s": round(plan_build_s, 3),
            "plan_scratch_bytes": {"forward": scratch[0]["partial_bytes"] + scratch[0]["padded_input_bytes"],
                                   "backward": scratch[1]["partial_bytes"] + scratch[1]["padded_input_bytes"],
                                   "of_which_padded_input_copy": scratch[0]["padded_input_bytes"]},
            "setup_s": round(setup_s, 2),
            "timed_path": "Python operator mirror: torch.empty_like output, accumulate=0, nts_spmm_gather_planned",
            "reference_operator": reference_operator,
        },
        "roofline": roofline,
        "check": check,
        "cpu_baseline": cpu_baseline,
        "epochs": epochs,
    }
    print(json.dumps(out))


def check_against_oracle(torch, chunk, inputs, outputs, V, n_rows=400, n_hubs=4):
    """The outputs of the last timed step against the CPU oracle: n_rows seeded rows per pass (rows that
    the schedule never cuts must equal the oracle's fused chain bit for bit, the others within 1e-4 of
    max(|a|, |b|, 1e-2 * sum|terms|)), and the n_hubs longest rows against a float64 sum -- the oracle's
    strictly sequential fp32 chain over 10^5..10^6 edges is itself several 1e-4 off there, so for those
    rows the kernel has to meet the tolerance against float64 and must not be less accurate than the
    oracle."""
    import numpy as np

    import oracle
    from neutronbench_amd import synth
    from neutronbench_amd.layout import u32_to_i64

    rows = synth.permutation(V, 7, chunk.column_offset_gpu.device)[:n_rows]
    worst, worst_hub, exact_rows, checked = 0.0, 0.0, 0, 0
    detail = {}
    for name, x in inputs.items():
        out = outputs[name]
        fwd = name.startswith("fwd")
        off = chunk.column_offset_gpu if fwd else chunk.row_offset_gpu
        idx = chunk.row_indices_gpu if fwd else chunk.column_indices_gpu
        w = chunk.edge_weight_forward_gpu if fwd else chunk.edge_weight_backward_gpu
        off64 = u32_to_i64(off)
        deg = off64[1:] - off64[:-1]
        hubs = torch.topk(deg, n_hubs).indices
        xh = x.cpu().numpy()

        def sub(sel):
            starts = off64[sel]
            lens = off64[sel + 1] - starts
            so = torch.zeros(sel.numel() + 1, dtype=torch.int64, device=off.device)
            so[1:] = torch.cumsum(lens, 0)
            eid = torch.repeat_interleave(starts - so[:-1], lens) + torch.arange(int(so[-1]), device=off.device)
            return so.cpu().numpy().astype(np.uint32), eid

        def err(a, b, scale):
            den = np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-2 * scale + 1e-30)
            return float((np.abs(a.astype(np.float64) - b) / den).max())

        so, eid = sub(rows)
        si, sw = idx[eid].cpu().numpy().view(np.uint32), w[eid].cpu().numpy()
        got = out[rows].cpu().numpy()
        ref = oracle.spmm(xh, sw, so, si, rows.numel())
        scale = oracle.spmm(np.abs(xh), sw, so, si, rows.numel())
        uncut = np.diff(so.astype(np.int64)) <= 128  # rows of at most chunk/4 edges are never cut
        fused = oracle.spmm(xh, sw, so, si, rows.numel(), fused=True)
        bits_ok = bool(np.array_equal(got[uncut].view(np.uint32), fused[uncut].view(np.uint32)))
        e_rows = err(got, ref, scale)
        ho, heid = sub(hubs)
        hi64, hw = u32_to_i64(idx[heid]), w[heid]
        exact = np.zeros((n_hubs, x.shape[1]))
        for k in range(n_hubs):
            acc = torch.zeros(x.shape[1], dtype=torch.float64, device=x.device)
            for s in range(int(ho[k]), int(ho[k + 1]), 1 << 15):
                e = min(s + (1 << 15), int(ho[k + 1]))
                acc += (x[hi64[s:e]].double() * hw[s:e, None].double()).sum(0)
            exact[k] = acc.cpu().numpy()
        hscale = oracle.spmm(np.abs(xh), hw.cpu().numpy(), ho, idx[heid].cpu().numpy().view(np.uint32), n_hubs)
        href = oracle.spmm(xh, hw.cpu().numpy(), ho, idx[heid].cpu().numpy().view(np.uint32), n_hubs)
        e_hub, e_hub_oracle = err(out[hubs].cpu().numpy(), exact, hscale), err(href, exact, hscale)
        detail[name] = {"rows_max_rel_err": e_rows, "uncut_rows_bit_exact": bits_ok, "uncut_rows": int(uncut.sum()),
                        "hub_max_rel_err_vs_f64": e_hub, "oracle_hub_max_rel_err_vs_f64": e_hub_oracle}
        worst, worst_hub = max(worst, e_rows), max(worst_hub, e_hub)
        exact_rows += int(uncut.sum()) if bits_ok else 0
        checked += rows.numel() + n_hubs
        if not bits_ok or e_rows > 1e-4 or e_hub > 1e-4 or e_hub > max(e_hub_oracle, 1e-5):
            return {"ok": False, "failed_pass": name, "detail": detail}
    return {"ok": True, "checked_rows": checked, "max_rel_err": worst, "bit_exact_rows": exact_rows,
            "hub_rows_max_rel_err_vs_f64": worst_hub, "tolerance": 1e-4,
            "note": "sampled rows of all four timed passes against the CPU oracle; the longest rows of each pass are "
                    "held to float64 (the oracle's sequential fp32 chain is less accurate there than the kernel)",
            "detail": detail}


def run_reference_programs(torch, chunk, x0, h1, V, sample_edges, reps):
    """The reference's own operators on the same graph, from the programs oracle/build_ref.sh builds out
    of the reference tree: ForwardCPUfuseOp on this host's cores (its loader, partitioner and operator
    unchanged) -> the CPU baseline; and ForwardSingleGPUfuseOp, the reference's GPU operator class
    compiled unchanged against this library's host veneer (torch::zeros output, accumulate = 1, the
    operator's own stream synchronisation) -> what an unchanged caller gets, outside the timed region.
    Returns (cpu_baseline or None, reference_operator or None)."""
    import re
    import shutil
    import subprocess
    import tempfile

    if not os.path.exists(REFERENCE_PROGRAM):
        return None, None
    E = chunk.E
    tmp = tempfile.mkdtemp(prefix="nts_ref_")
    cpu = gpu = None
    try:
        ro = chunk.row_offset_gpu.to(torch.int64)
        pos = torch.arange(sample_edges, device=ro.device)
        src = torch.searchsorted(ro, pos, right=True) - 1
        dst = chunk.column_indices_gpu[:sample_edges].to(torch.int64)
        torch.stack([src, dst], 1).to(torch.int32).cpu().numpy().tofile(os.path.join(tmp, "g.edge"))
        del ro, pos, src, dst
        x0.cpu().numpy().tofile(os.path.join(tmp, f"p.x{F_IN}"))
        h1.cpu().numpy().tofile(os.path.join(tmp, f"p.x{F_HID}"))
        env = dict(os.environ, NTS_REF_WARMUP="1", NTS_REF_REPS=str(reps))
        pat = (r"timing: V=\d+ E=(\d+) F=(\d+) forward_s=([0-9.]+) backward_s=([0-9.]+)(?: threads=(\d+))? "
               r"best_forward_s=([0-9.]+) best_backward_s=([0-9.]+)")
        argv = [os.path.join(tmp, "g.edge"), str(V), f"{F_IN},{F_HID}", "1", os.path.join(tmp, "p")]
        r = subprocess.run([REFERENCE_PROGRAM] + argv + ["agg-cpu"], capture_output=True, text=True, timeout=400, env=env)
        rows = re.findall(pat, r.stdout)
        if r.returncode == 0 and len(rows) == 2:
            total_s = sum(float(f) + float(b) for _, _, f, b, _, _, _ in rows)
            edges = int(rows[0][0])
            cpu = {
                "value": round(4 * edges / total_s, 1),
                "unit": "edges/s",
                "cores": int(rows[0][4]),
                "kind": "reference",
                "sample": f"the reference's ForwardCPUfuseOp (its own loader, partitioner and operator, built from the "
                          f"reference sources) on {'the whole graph' if edges == E else 'the lowest-numbered source vertices'}"
                          f" ({edges} edges), forward and backward at F={F_IN} and F={F_HID}, median of {reps} after 1 "
                          f"warm-up, {rows[0][4]} threads (the operator's only setting: every configured CPU): "
                          + ", ".join(f"F={w} fwd {float(f):.3f} s bwd {float(b):.3f} s" for _, w, f, b, _, _, _ in rows),
            }
        if os.path.exists(REFERENCE_GPU_PROGRAM):
            r = subprocess.run([REFERENCE_GPU_PROGRAM] + argv + ["agg-gpu"], capture_output=True, text=True, timeout=400,
                               env=env)
            rows = re.findall(pat, r.stdout)
            if r.returncode == 0 and len(rows) == 2:
                gpu = {"what": "the reference's ForwardSingleGPUfuseOp class, unchanged, over the host veneer "
                               "(torch::zeros output, zero_buffer, the aggregation, stream synchronisation per call; the veneer "
                               "writes into the output it has just seen cleared and checks its schedule on a side stream); wall time per "
                               f"call, median of {reps} after 1 warm-up; the veneer builds its schedule on the third "
                               "identical call, so the best time is the steady state",
                       "edges": int(rows[0][0])}
                for _, w, f, b, _, bf, bb in rows:
                    gpu[f"F{w}_forward_ms"] = round(float(f) * 1e3, 3)
                    gpu[f"F{w}_backward_ms"] = round(float(b) * 1e3, 3)
                    gpu[f"F{w}_best_forward_ms"] = round(float(bf) * 1e3, 3)
                    gpu[f"F{w}_best_backward_ms"] = round(float(bb) * 1e3, 3)
    except (OSError, subprocess.SubprocessError):
        pass
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return cpu, gpu


def run_cpu_port_baseline(torch, chunk, x0, h1, g1, g0, V, reps):
    """The CPU oracle (restatement of the reference's CPU operators, OpenMP over rows) on the whole graph,
    the four passes of a step, at the two thread settings the reference uses: every hardware thread
    (its full-graph operators) and max(1, ncpu / 2 - 1) (its sampler's default, core/coocsc.hpp:50).
    Median of `reps` after one warm-up each."""
    import numpy as np

    import oracle
    from neutronbench_amd.layout import u32_to_i64

    all_threads = oracle.max_threads()
    co = u32_to_i64(chunk.column_offset_gpu).cpu().numpy().astype(np.uint32)
    ro = u32_to_i64(chunk.row_offset_gpu).cpu().numpy().astype(np.uint32)
    fi = chunk.row_indices_gpu.cpu().numpy().view(np.uint32)
    bi = chunk.column_indices_gpu.cpu().numpy().view(np.uint32)
    fw, bw = chunk.edge_weight_forward_gpu.cpu().numpy(), chunk.edge_weight_backward_gpu.cpu().numpy()
    xs = [t.cpu().numpy() for t in (x0, h1, g1, g0)]
    E = chunk.E

    def one(threads):
        t = time.perf_counter()
        oracle.spmm(xs[0], fw, co, fi, V, threads=threads)
        oracle.spmm(xs[1], fw, co, fi, V, threads=threads)
        oracle.spmm(xs[2], bw, ro, bi, V, threads=threads)
        oracle.spmm(xs[3], bw, ro, bi, V, threads=threads)
        return time.perf_counter() - t

    out = {}
    for key, threads in (("all_threads", all_threads), ("reference_default_threads", max(1, all_threads // 2 - 1))):
        one(threads)
        times = sorted(one(threads) for _ in range(reps))
        med = times[len(times) // 2] if len(times) % 2 else 0.5 * (times[len(times) // 2 - 1] + times[len(times) // 2])
        out[key] = {"value": round(4 * E / med, 1), "unit": "edges/s", "cores": threads, "kind": "port",
                    "sample": f"the CPU oracle on the whole graph ({E} edges), four passes (F=602 and F=128, forward "
                              f"and backward), median of {reps} after 1 warm-up: {med:.3f} s per step"}
    return out


def run_epochs(torch, names, with_cpu, cpu_batches):
    """One epoch of each sampled mini-batch configuration, driven from C++ through the C ABI
    (neutronbench_amd/host/epoch_driver.cpp -> lib/nts_epoch; sampling, layer construction,
    feature/label gather, aggregation forward + backward of every layer; dense layers are not part of
    this library).  Per configuration: the serial epoch -- one stream, a wait after every stage, the
    figure and the stage columns of the reference's log line (toolkits/GCN_GPU_NEIGHBOR.hpp:1498-1506) --
    the same epoch with four batches in flight, a check of every array of one batch of the epoch
    against the CPU oracle (oracle/epoch_check.py), and the CPU oracle timed on a few batches."""
    import shutil
    import tempfile

    from neutronbench_amd import epoch
    from oracle import epoch_check

    records = {}
    written = {}  # inputs on disk, shared by the configurations on the same graph (products, gat)
    try:
        for name in names:
            cfg = epoch.CONFIGS[name]
            key = tuple(cfg[k] for k in ("V", "E", "F", "seed", "classes", "train"))
            if key not in written:
                for d, _ in written.values():
                    shutil.rmtree(d, ignore_errors=True)
                written.clear()
                d = tempfile.mkdtemp(prefix="nts_epoch_")
                written[key] = (d, epoch.write_native_inputs(name, d, keep_host=True))
            d, host = written[key]
            dump = tempfile.mkdtemp(prefix="nts_dump_")
            try:
                serial = epoch.run_native_on(d, name, host["V"], pipeline=1, stage_sync=True, dump_dir=dump,
                                             dump_batch=1)
                piped = epoch.run_native_on(d, name, host["V"], pipeline=4, stage_sync=False)
                check = epoch_check.check_dump(dump, host["co"], host["ri"], host["feat"], host["labels"], cfg["fanout"],
                                               cfg["cache"]) if with_cpu else None
            finally:
                shutil.rmtree(dump, ignore_errors=True)
            cpu = epoch_cpu_baseline(torch, name, host, serial["batches"], cpu_batches) if with_cpu else None
            if cpu is not None and not cfg.get("heads"):
                cpu["reference_sampler_and_operator"] = epoch_reference_cpu(name, host, serial["batches"], cpu_batches)
            records[name] = {
                "epoch_s": serial["epoch_s"], "stage_s": serial.get("stage_s"), "batches": serial["batches"],
                "batch_size": cfg["batch"], "fanout_output_side_first": cfg["fanout"], "heads": cfg.get("heads", 0),
                "vertices": host["V"], "edges": host["E"], "sampled_edges": serial["sampled_edges"],
                "gathered_rows": serial["gathered_rows"], "cache_hit_rate": serial.get("cache_hit_rate"),
                "ms_per_batch": round(1e3 * serial["epoch_s"] / max(serial["batches"], 1), 4),
                "pipelined_epoch_s": piped["epoch_s"], "pipeline_depth": piped["pipeline"],
                "driver": "lib/nts_epoch (C++ over the C ABI), one stream, a wait after every stage; 2 untimed batches first",
                # how the whole-batch builder replays its launches (nts_batch_builder_use_graph): 2 = the hops'
                # transpositions on a side branch of its graph, 3 = as a second graph beside the feature gather
                # (sample time is then the sampling alone); the pipelined run: 1 = one chain
                "hop_graph_mode": serial.get("hop_graph_mode"), "pipelined_hop_graph_mode": piped.get("hop_graph_mode"),
                # the program asks the HIP runtime for eight hardware queues when four batches are in flight
                "pipelined_hw_queues": 8 if piped["pipeline"] == 4 else None,
                "check": check, "cpu_baseline": cpu,
            }
    finally:
        for d, _ in written.values():
            shutil.rmtree(d, ignore_errors=True)
    return records


def run_epoch_workload(args):
    """Per-epoch time of one sampled mini-batch configuration (see run_epochs) as a JSON line of its own:
    `value` is the serial epoch time, config.pipelined_epoch_s the time with four batches in flight."""
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP library has no CPU fallback)")
    rec = run_epochs(torch, (args.workload,), not args.no_cpu_baseline, args.cpu_batches)[args.workload]
    if rec["check"] is not None and not rec["check"]["ok"]:
        print(json.dumps({"error": "a batch of the epoch differs from the CPU oracle", "check": rec["check"]}))
        sys.exit(1)
    line = {
        "metric": "epoch time", "value": rec["epoch_s"], "unit": "s", "n_gpus": 1, "steps": rec["batches"],
        "warmup": 2, "ms_per_step": rec["ms_per_batch"],
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}-shaped sampled mini-batch epoch, fanout (output side first) "
                               f"{rec['fanout_output_side_first']}, batch {rec['batch_size']}, {rec['batches']} batches; "
                               "a step = one batch: sampling, layer construction, feature/label gather, aggregation "
                               "fwd+bwd of every layer",
                   **{k: rec[k] for k in ("vertices", "edges", "stage_s", "sampled_edges", "gathered_rows",
                                          "cache_hit_rate", "pipelined_epoch_s", "pipeline_depth", "driver",
                                          "hop_graph_mode", "pipelined_hop_graph_mode")}},
        "roofline": None,
        "check": rec["check"],
        "cpu_baseline": rec["cpu_baseline"],
    }
    print(json.dumps(line))


def epoch_reference_cpu(name, host, n_batches, k_batches):
    """The reference's own host side of a mini-batch -- Sampler::sample_one (neighbour pick, relabelling,
    CSR, weights) and MiniBatchFuseOp forward + backward of every layer -- timed by oracle/_ref/ref_minibatch
    on k batches of the same graph (its loader reads the edge list this function writes), extrapolated to
    the epoch.  None when the program has not been built (no reference tree) or fails."""
    import re
    import shutil
    import subprocess
    import tempfile

    import numpy as np

    from neutronbench_amd import epoch

    if not os.path.exists(REFERENCE_MINIBATCH_PROGRAM):
        return None
    cfg = epoch.CONFIGS[name]
    V = host["V"]
    tmp = tempfile.mkdtemp(prefix="nts_refmb_")
    try:
        owner = np.repeat(np.arange(V, dtype=np.uint32), np.diff(host["co"].astype(np.int64)))
        np.stack([host["ri"], owner], 1).astype(np.uint32).tofile(os.path.join(tmp, "g.edge"))
        del owner
        layers = "-".join(map(str, [cfg["F"]] + [cfg["hidden"]] * (len(cfg["fanout"]) - 1) + [cfg["classes"]]))
        fan = ",".join(map(str, reversed(cfg["fanout"])))  # the reference reverses its FANOUT string
        lines = dict(ALGORITHM="GCNNEIGHBORGPU", VERTICES=V, EPOCHS=1, LAYERS=layers, FANOUT=fan, VALFANOUT=fan,
                     BATCH_SIZE=cfg["batch"], BATCH_TYPE="shuffle", EDGE_FILE=f"{tmp}/g.edge", FEATURE_FILE="none",
                     LABEL_FILE="none", MASK_FILE="none", MINI_PULL=1, CACHE_TYPE="none", PIPELINES=1, MODE="pipeline",
                     CLASSES=1, PROC_OVERLAP=0, PROC_LOCAL=0, PROC_CUDA=0, PROC_REP=0, LOCK_FREE=1, TIME_SKIP=0, RUNS=1,
                     LEARN_RATE=0.01, WEIGHT_DECAY=0.0001, DECAY_RATE=0.97, DECAY_EPOCH=100, DROP_RATE=0.5)
        with open(os.path.join(tmp, "g.cfg"), "w") as f:
            f.write("".join(f"{k}:{v}\n" for k, v in lines.items()))
        t0 = time.perf_counter()
        r = subprocess.run([REFERENCE_MINIBATCH_PROGRAM, os.path.join(tmp, "g.cfg"), str(k_batches), "time"],
                           capture_output=True, text=True, timeout=300, cwd=tmp)
        wall = time.perf_counter() - t0
        m = re.search(r"reference mini-batch cpu timing: batches=(\d+) sample_s=([0-9.]+) aggregate_s=([0-9.]+) "
                      r"sampled_edges=(\d+) threads=(\d+)", r.stdout)
        if r.returncode != 0 or not m or int(m.group(1)) == 0:
            return None
        k, ts, ta = int(m.group(1)), float(m.group(2)), float(m.group(3))
        return {"value": round((ts + ta) / k * n_batches, 4), "unit": "s", "cores": int(m.group(5)), "kind": "reference",
                "sample": f"the reference's Sampler::sample_one and MiniBatchFuseOp (forward + backward of every layer) on "
                          f"{k} batches of {cfg['batch']} after one untimed batch, on its own loader's copy of the graph, "
                          f"extrapolated to {n_batches} batches: per batch sampling {ts / k * 1e3:.2f} ms, aggregation "
                          f"{ta / k * 1e3:.2f} ms ({int(m.group(4)) // k} sampled edges); the feature gather is not "
                          f"included; built with the METIS shim of oracle/build_toolkits.sh; program wall time {wall:.1f} s"}
    except (OSError, subprocess.SubprocessError):
        return None
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def epoch_cpu_baseline(torch, name, host, n_batches, k_batches):
    """The CPU oracle (restatement of the reference's host steps: sampCSC::postprocessing,
    generate_csr_from_csc, update_degree + compute_weight_*, get_feature, MiniBatchFuseOp forward and
    backward; for the GAT configuration the chain of the reference's CPU edge operators,
    toolkits/GAT_CPU.hpp:178-204) on the first k batches of the epoch, extrapolated to the epoch.  The
    neighbour pick itself is an input here (the lists the library sampled are used), so the reference's
    CPU sampling time is not part of the figure."""
    import numpy as np

    import oracle
    from neutronbench_amd import epoch
    from neutronbench_amd.batch import BatchBuilder

    cfg = epoch.CONFIGS[name]
    dev = torch.device("cuda:0")
    V = host["V"]
    gco = torch.from_numpy(host["co"].view(np.int32)).to(dev)
    gri = torch.from_numpy(host["ri"].view(np.int32)).to(dev)
    feat = host["feat"]
    train32 = torch.from_numpy(host["train"].view(np.int32)).to(dev)
    heads = cfg.get("heads", 0)
    builder = BatchBuilder(gco, gri, cfg["fanout"], cfg["batch"], want_perm=heads > 0)
    threads = oracle.max_threads()
    rng = np.random.default_rng(1)
    t = {"structure": 0.0, "gather": 0.0, "aggregate": 0.0}
    k_batches = max(1, min(k_batches, n_batches))
    u32 = lambda a: a.cpu().numpy().view(np.uint32)  # noqa: E731
    # Batch 0 runs once more in front, untimed: the first call starts the oracle's worker threads and
    # touches its buffers' pages for the first time, which is not what a batch of an epoch costs.
    for turn, b in enumerate([0] + list(range(k_batches))):
        if turn == 1:
            t = dict.fromkeys(t, 0.0)
        layers = builder.sample(train32[b * cfg["batch"]:(b + 1) * cfg["batch"]], 1000 * b)
        hostl = [dict(dst=u32(l.dev_destination), co=u32(l.dev_column_offset), src=u32(l.dev_source),
                      glob=u32(l.dev_source)[u32(l.dev_row_indices)]) for l in layers]
        outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
        built = []
        t0 = time.perf_counter()
        for h in hostl[::-1]:  # hop order: the batch's own hop first
            local, source, n = oracle.postprocess(h["glob"], V)
            ro, ci = oracle.csr_from_csc(h["co"], local, n)
            ewf, ewb = oracle.layer_weights(h["co"], local, ro, ci, source, h["dst"], outd, ind)
            built.append((h["co"], local, ro, ci, ewf, ewb, h["dst"].size, n))
        t["structure"] += time.perf_counter() - t0
        built = built[::-1]  # input side first
        t0 = time.perf_counter()
        x = oracle.get_feature(feat, hostl[0]["src"])
        t["gather"] += time.perf_counter() - t0
        widths = [cfg["F"]] + [cfg["hidden"]] * (len(built) - 1)
        for (lco, local, ro, ci, ewf, ewb, Vd, Vs), F in zip(built, widths):
            if heads:
                H, Fh = heads, cfg["hidden"] // heads
                E = local.size
                xin = rng.standard_normal((Vs, H * Fh)).astype(np.float32)
                el = rng.standard_normal((Vs, H)).astype(np.float32)
                er = np.zeros((Vd, H), np.float32)
                g = rng.standard_normal((Vd, H * Fh)).astype(np.float32)
                t0 = time.perf_counter()
                pre = oracle.scatter_src(el, lco, local) + oracle.scatter_dst(er, lco, E)
                alpha = oracle.edge_softmax(np.where(pre > 0, pre, np.float32(0.2) * pre), lco)
                msg = oracle.scatter_src(xin, lco, local)
                x = oracle.aggregate_dst((msg.reshape(E, H, Fh) * alpha[:, :, None]).reshape(E, H * Fh), lco)
                gmsg = oracle.scatter_dst(g, lco, E)
                oracle.gather_to_src((gmsg.reshape(E, H, Fh) * alpha[:, :, None]).reshape(E, H * Fh), lco, local, Vs)
                galpha = (msg.reshape(E, H, Fh) * gmsg.reshape(E, H, Fh)).sum(2)
                gs = oracle.edge_softmax_bwd(galpha, alpha, lco) * np.where(pre > 0, np.float32(1), np.float32(0.2))
                oracle.aggregate_dst(gs, lco)
                oracle.gather_to_src(gs, lco, local, Vs)
                t["aggregate"] += time.perf_counter() - t0
                continue
            xin = x if x.shape == (Vs, F) else rng.standard_normal((Vs, F)).astype(np.float32)
            g = rng.standard_normal((Vd, F)).astype(np.float32)
            t0 = time.perf_counter()
            x = oracle.spmm(xin, ewf, lco, local, Vd, threads=threads)
            oracle.spmm(g, ewb, ro, ci, Vs, threads=threads)
            t["aggregate"] += time.perf_counter() - t0
    builder.close()
    del gco, gri
    per_batch = sum(t.values()) / k_batches
    return {
        "value": round(per_batch * n_batches, 4), "unit": "s", "cores": threads, "kind": "port",
        "sample": f"the CPU oracle on the first {k_batches} of {n_batches} batches (the library's sampled neighbour "
                  f"lists as input; the neighbour pick itself is not timed; one untimed batch first), extrapolated "
                  f"to the epoch: per batch "
                  + ", ".join(f"{k} {v / k_batches * 1e3:.2f} ms" for k, v in t.items()),
    }


if __name__ == "__main__":
    main()
