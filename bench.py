#!/usr/bin/env python3
"""Benchmark of the aggregation hot path on one MI355X.

Workload (BASELINE.json configs[2]): Reddit-shaped full-graph 2-layer GCN aggregation,
forward + backward, whole graph resident in HBM.  232,965 vertices, 114.8 M directed R-MAT edges,
GCN-normalised edge weights, fp32.  One step = the four aggregations of one training iteration in
aggregate-then-transform order: layer-0 forward (F=602), layer-1 forward (F=128), layer-1 backward
(F=128), layer-0 backward (F=602).  Forward gathers by destination over the CSC, backward gathers
by source over the CSR.  Inputs are resident in HBM before the timed region.

Prints one JSON line: edges aggregated per second (4 * E edges per step), the roofline figure of
the dominant kernel (the F=602 gather) from HIP events recorded around that kernel, and a CPU
baseline timed on the host cores on a bounded sample of the same graph: the reference's own CPU
operator where the reference-built program oracle/_ref/ref_fullgraph_cpu is present ("reference"),
else the CPU oracle ("port").

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
# The reference's own CPU operator, built from the reference tree where that is present (test infrastructure).
REFERENCE_PROGRAM = os.path.join(ROOT, "oracle", "_ref", "ref_fullgraph_cpu")
HBM_PEAK_GBS = 8000.0
# Bytes per launch of the F=602 gather kernel that cross the L2 <-> fabric boundary, from rocprofv3
# FETCH_SIZE (x1.986 calibration) + WRITE_SIZE at the default schedule
# (profiles/spmm_wave_f602_reddit_shaped_pmc.txt).  Reported only for the configuration it was measured on.
TRAFFIC_BYTES_F602 = 44_601_740_400
TRAFFIC_MEASURED_AT = dict(vertices=V_REDDIT, edges=E_REDDIT, chunk=512, slabs=32)


def algorithmic_bytes(E, V_out, F, weighted=True):
    """Edge-gather model of one aggregation pass: one source row, one index and one weight per
    edge; one output row and one offset per output row."""
    return E * (4 * F + 4 + (4 if weighted else 0)) + V_out * 4 * F + (V_out + 1) * 4


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
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one plain 1 GiB row copy (identity gather) so that HBM byte counters can be scaled")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the oracle sample")
    ap.add_argument("--cpu-reference-edges", type=int, default=28_700_000,
                    help="edges of the sample the reference's own CPU operator is timed on (0 = time the oracle instead)")
    ap.add_argument("--workload", choices=["reddit", "arxiv", "products", "gat"], default="reddit",
                    help="reddit (default): the aggregation workload above; arxiv / products / gat: per-epoch time of "
                         "that sampled mini-batch configuration (BASELINE.json configs 2, 4, 5) instead")
    ap.add_argument("--cpu-batches", type=int, default=3, help="mini-batch workloads: batches the CPU oracle is timed on")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")
    if args.workload != "reddit":
        return run_epoch_workload(args)

    import torch

    from neutronbench_amd import synth
    from neutronbench_amd.abi import call, ptr
    from neutronbench_amd.layout import FullGraphChunk
    from neutronbench_amd.ops import ForwardSingleGPUfuseOp

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP library has no CPU fallback)")
    dev = torch.device("cuda:0")
    V, E = args.vertices, args.edges

    t0 = time.time()
    src, dst = synth.rmat_edges(V, E, 0.57, 0.19, 0.19, seed=3, device=dev, sort=True)
    chunk = FullGraphChunk.from_edges(src, dst, V, args.chunk, args.slabs)
    del src, dst
    x0 = synth.normal_features(V, F_IN, seed=31, device=dev)
    h1 = synth.normal_features(V, F_HID, seed=32, device=dev)
    g1 = synth.normal_features(V, F_HID, seed=33, device=dev)
    g0 = synth.normal_features(V, F_IN, seed=34, device=dev)
    torch.cuda.synchronize()
    setup_s = time.time() - t0
    op = ForwardSingleGPUfuseOp(chunk, with_weight=True)
    chunk.plan_forward.reserve(F_IN)
    chunk.plan_backward.reserve(F_IN)

    def step():
        y0 = op.forward(x0)    # layer 0: aggregate the 602-wide input features
        y1 = op.forward(h1)    # layer 1: aggregate the 128-wide hidden features
        d1 = op.backward(g1)   # layer 1 backward: gradient gather over the CSR
        d0 = op.backward(g0)   # layer 0 backward
        return y0, y1, d1, d0

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

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # One HIP event pair per aggregation launch of the timed region (4 per step).  The library records
    # them on the launch stream immediately before and after its main gather kernel; nothing waits on
    # them until the timed region is over.
    stream = torch.cuda.current_stream().cuda_stream
    n_ev = 4 * args.steps
    events = []
    for _ in range(n_ev):
        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        call("nts_event_create", ctypes.byref(a))
        call("nts_event_create", ctypes.byref(b))
        events.append((a, b))
    fwd, bwd = chunk.plan_forward.handle, chunk.plan_backward.handle

    def timed_step(i):
        call("nts_spmm_plan_set_events", fwd, *events[4 * i + 0])
        op.forward(x0)
        call("nts_spmm_plan_set_events", fwd, *events[4 * i + 1])
        op.forward(h1)
        call("nts_spmm_plan_set_events", bwd, *events[4 * i + 2])
        op.backward(g1)
        call("nts_spmm_plan_set_events", bwd, *events[4 * i + 3])
        op.backward(g0)

    # Timed region: exactly `steps` steps between two synchronisations.
    torch.cuda.synchronize()
    t_start = time.perf_counter()
    for i in range(args.steps):
        timed_step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_start
    ms_per_step = elapsed * 1e3 / args.steps
    edges_per_s = 4.0 * E / (elapsed / args.steps)
    call("nts_spmm_plan_set_events", fwd, None, None)
    call("nts_spmm_plan_set_events", bwd, None, None)

    durs = []
    for a, b in events:
        ms = ctypes.c_float()
        call("nts_event_elapsed_ms", ctypes.byref(ms), a, b)
        durs.append(ms.value)
        call("nts_event_destroy", a)
        call("nts_event_destroy", b)
    per_pass = [sum(durs[k::4]) / args.steps for k in range(4)]  # fwd602, fwd128, bwd128, bwd602
    # Dominant kernel: the F=602 gather (spmm_wave_kernel<1,10>), launched twice per step: forward
    # over the CSC and backward over the CSR.  Same algorithmic bytes per launch for both.
    kernel_ms = (per_pass[0] + per_pass[3]) / 2
    algo = algorithmic_bytes(E, V, F_IN)
    achieved = algo / (kernel_ms * 1e-3) / 1e9
    roofline = {
        "bound": "hbm",
        "kernel": "spmm_wave_kernel<1,10,true,false,false> (F=602 gather, forward and backward launches)",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": TRAFFIC_BYTES_F602 if dict(vertices=V, edges=E, chunk=args.chunk, slabs=args.slabs) ==
        TRAFFIC_MEASURED_AT else None,
        "algorithmic_bytes": algo,
        "kernel_ms": round(kernel_ms, 3),
        "per_pass_ms": {"fwd_F602": round(per_pass[0], 3), "fwd_F128": round(per_pass[1], 3),
                        "bwd_F128": round(per_pass[2], 3), "bwd_F602": round(per_pass[3], 3)},
    }

    cpu_baseline = None
    if not args.no_cpu_baseline:
        if args.cpu_reference_edges > 0 and os.path.exists(REFERENCE_PROGRAM):
            cpu_baseline = run_reference_cpu_baseline(torch, chunk, x0, h1, V, min(E, args.cpu_reference_edges))
        if cpu_baseline is None:
            cpu_baseline = run_cpu_baseline(torch, chunk, x0, h1, g1, g0, V, args.cpu_seconds)

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
            "graph": "R-MAT a=.57 b=.19 c=.19, seed 3, ids permuted, edge list in (src, dst) order, duplicates kept",
            "passes_per_step": 4,
            "plan": dict(chunk.plan_forward.info(), chunk_edges=args.chunk, slabs=args.slabs),
            "setup_s": round(setup_s, 2),
        },
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
    }
    print(json.dumps(out))


def run_reference_cpu_baseline(torch, chunk, x0, h1, V, sample_edges):
    """The reference's own CPU operator (ForwardCPUfuseOp behind oracle/_ref/ref_fullgraph_cpu, built
    from the reference tree by oracle/build_ref.sh) on the edges of the lowest-numbered source
    vertices of the same graph: its loader, partitioner and operator run unchanged on this host's
    cores.  Returns None when the program fails, so that the caller can fall back to the oracle."""
    import re
    import shutil
    import subprocess
    import tempfile

    tmp = tempfile.mkdtemp(prefix="nts_ref_")
    try:
        ro = chunk.row_offset_gpu.to(torch.int64)
        pos = torch.arange(sample_edges, device=ro.device)
        src = torch.searchsorted(ro, pos, right=True) - 1
        dst = chunk.column_indices_gpu[:sample_edges].to(torch.int64)
        torch.stack([src, dst], 1).to(torch.int32).cpu().numpy().tofile(os.path.join(tmp, "g.edge"))
        del ro, pos, src, dst
        x0.cpu().numpy().tofile(os.path.join(tmp, f"p.x{F_IN}"))
        h1.cpu().numpy().tofile(os.path.join(tmp, f"p.x{F_HID}"))
        r = subprocess.run([REFERENCE_PROGRAM, os.path.join(tmp, "g.edge"), str(V), f"{F_IN},{F_HID}", "1",
                            os.path.join(tmp, "p"), "agg-cpu"], capture_output=True, text=True, timeout=240)
        rows = re.findall(r"timing: V=\d+ E=(\d+) F=(\d+) forward_s=([0-9.]+) backward_s=([0-9.]+) threads=(\d+)", r.stdout)
        if r.returncode != 0 or len(rows) != 2:
            return None
        total_s = sum(float(f) + float(b) for _, _, f, b, _ in rows)
        edges = int(rows[0][0])
        return {
            "value": round(4 * edges / total_s, 1),
            "unit": "edges/s",
            "cores": int(rows[0][4]),
            "kind": "reference",
            "sample": f"the reference's ForwardCPUfuseOp (its own loader, partitioner and operator, built from the "
                      f"reference sources) on the {edges} edges of the lowest-numbered source vertices of the same "
                      f"graph, forward and backward at F={F_IN} and F={F_HID}, best of 3: "
                      + ", ".join(f"F={w} fwd {float(f):.3f} s bwd {float(b):.3f} s" for _, w, f, b, _ in rows),
        }
    except (OSError, subprocess.SubprocessError):
        return None
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def run_cpu_baseline(torch, chunk, x0, h1, g1, g0, V, target_s):
    """The CPU oracle (restatement of the reference's CPU operators, OpenMP over rows) on the first
    R output rows of each of the four passes of the same graph, all host cores."""
    import numpy as np

    import oracle
    from neutronbench_amd.layout import u32_to_i64

    threads = oracle.max_threads()
    co = u32_to_i64(chunk.column_offset_gpu).cpu().numpy()
    ro = u32_to_i64(chunk.row_offset_gpu).cpu().numpy()
    xs = [t.cpu().numpy() for t in (x0, h1, g1, g0)]

    def slice_rows(offsets, indices_dev, weights_dev, rows):
        e = int(offsets[rows])
        idx = indices_dev[:e].cpu().numpy().view(np.uint32)
        w = weights_dev[:e].cpu().numpy()
        return offsets[: rows + 1].astype(np.uint32), idx, w, e

    def run(rows):
        fo, fi, fw, fe = slice_rows(co, chunk.row_indices_gpu, chunk.edge_weight_forward_gpu, rows)
        bo, bi, bw, be = slice_rows(ro, chunk.column_indices_gpu, chunk.edge_weight_backward_gpu, rows)
        t = time.perf_counter()
        oracle.spmm(xs[0], fw, fo, fi, rows, threads=threads)
        oracle.spmm(xs[1], fw, fo, fi, rows, threads=threads)
        oracle.spmm(xs[2], bw, bo, bi, rows, threads=threads)
        oracle.spmm(xs[3], bw, bo, bi, rows, threads=threads)
        return time.perf_counter() - t, 2 * (fe + be)

    probe_rows = min(V, 512)
    t_probe, e_probe = run(probe_rows)
    rate = e_probe / max(t_probe, 1e-6)
    # rows whose four passes need about target_s at the probed rate
    want_edges = rate * target_s
    per_row = (co[V] + ro[V]) * 2 / V
    rows = int(max(probe_rows, min(V, want_edges / max(per_row, 1))))
    t_run, e_run = run(rows)
    return {
        "value": round(e_run / t_run, 1),
        "unit": "edges/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {rows} destination rows (forward) and first {rows} source rows (backward) of the same "
                  f"graph, F=602 and F=128, {e_run} edge visits in {t_run:.2f} s",
    }


def run_epoch_workload(args):
    """Per-epoch time of a sampled mini-batch configuration through the library (every stage through
    the C ABI, see neutronbench_amd/epoch.py), next to the CPU oracle on a few batches of the same
    epoch.  One JSON line; `value` is the epoch time with the stages run one after the other, as the
    reference's default mode does, and config.pipelined_epoch_s the time with four batches in flight
    (two being sampled, one gathered, one aggregated, each stage on streams of its own)."""
    import torch

    from neutronbench_amd import epoch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP library has no CPU fallback)")
    serial = epoch.run(args.workload, pipeline=1, quiet=True)
    piped = epoch.run(args.workload, pipeline=4, quiet=True)
    cpu = None
    if not args.no_cpu_baseline and args.workload != "gat":
        cpu = epoch_cpu_baseline(torch, args.workload, serial["batches"], args.cpu_batches)
    cfg = epoch.CONFIGS[args.workload]
    line = {
        "metric": "epoch time", "value": serial["epoch_s"], "unit": "s", "n_gpus": 1, "steps": serial["batches"],
        "warmup": serial["warmup_batches"], "ms_per_step": round(1e3 * serial["epoch_s"] / serial["batches"], 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}-shaped sampled mini-batch epoch, fanout (output side first) "
                               f"{cfg['fanout']}, batch {cfg['batch']}, {serial['batches']} batches; a step = one batch: "
                               "sampling, layer construction, feature/label gather, aggregation fwd+bwd of every layer",
                   "vertices": serial["vertices"], "edges": serial["edges"], "stage_s": serial["stage_s"],
                   "sampled_edges": serial["sampled_edges"], "gathered_rows": serial["gathered_rows"],
                   "cache_hit_rate": serial["cache_hit_rate"], "pipelined_epoch_s": piped["epoch_s"],
                   "pipeline_depth": piped["pipeline"]},
        "roofline": None,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


def epoch_cpu_baseline(torch, name, n_batches, k_batches):
    """The CPU oracle (restatement of the reference's host steps: sampCSC::postprocessing,
    generate_csr_from_csc, update_degree + compute_weight_*, get_feature, MiniBatchFuseOp forward and
    backward) on the first k batches of the epoch, extrapolated to the epoch.  The neighbour pick
    itself is an input here (the lists the library sampled are used), so the reference's CPU
    sampling time is not part of the figure."""
    import numpy as np

    import oracle
    from neutronbench_amd import epoch, synth
    from neutronbench_amd.batch import BatchBuilder
    from neutronbench_amd.layout import as_u32

    cfg = epoch.CONFIGS[name]
    dev = torch.device("cuda:0")
    V, E = cfg["V"], cfg["E"]
    src, dst = synth.rmat_edges(V, E, seed=cfg["seed"], device=dev, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    del src, dst
    gco, gri = as_u32(co), as_u32(ri)
    feat = synth.normal_features(V, cfg["F"], seed=cfg["seed"] + 40).numpy()
    train32 = as_u32(synth.permutation(V, cfg["seed"] + 42, dev)[:cfg["train"]])
    builder = BatchBuilder(gco, gri, cfg["fanout"], cfg["batch"])
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
        host = [dict(dst=u32(l.dev_destination), co=u32(l.dev_column_offset), src=u32(l.dev_source),
                     glob=u32(l.dev_source)[u32(l.dev_row_indices)]) for l in layers]
        outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
        built = []
        t0 = time.perf_counter()
        for h in host[::-1]:  # hop order: the batch's own hop first
            local, source, n = oracle.postprocess(h["glob"], V)
            ro, ci = oracle.csr_from_csc(h["co"], local, n)
            ewf, ewb = oracle.layer_weights(h["co"], local, ro, ci, source, h["dst"], outd, ind)
            built.append((h["co"], local, ro, ci, ewf, ewb, h["dst"].size, n))
        t["structure"] += time.perf_counter() - t0
        built = built[::-1]  # input side first
        t0 = time.perf_counter()
        x = oracle.get_feature(feat, host[0]["src"])
        t["gather"] += time.perf_counter() - t0
        widths = [cfg["F"]] + [cfg["hidden"]] * (len(built) - 1)
        for (lco, local, ro, ci, ewf, ewb, Vd, Vs), F in zip(built, widths):
            xin = x if x.shape == (Vs, F) else rng.standard_normal((Vs, F)).astype(np.float32)
            g = rng.standard_normal((Vd, F)).astype(np.float32)
            t0 = time.perf_counter()
            x = oracle.spmm(xin, ewf, lco, local, Vd, threads=threads)
            oracle.spmm(g, ewb, ro, ci, Vs, threads=threads)
            t["aggregate"] += time.perf_counter() - t0
    builder.close()
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
