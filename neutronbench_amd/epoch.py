"""Per-epoch time of the sampled mini-batch path with the stage breakdown of the reference's log
line (toolkits/GCN_GPU_NEIGHBOR.hpp:1498-1506): sample / structure / gather / aggregate forward /
aggregate backward.  Dense layers are not part of this library and are left out.

    python -m neutronbench_amd.epoch --config arxiv|products|gat [--scale S]

Configurations (BASELINE.json configs 2, 4, 5).  Fanouts are listed in hop order, the batch's own hop
first: the reference reverses its FANOUT string ("10,25" for the first one) and gives entry i to hop i
(toolkits/GCN_GPU_NEIGHBOR.hpp:126-130, core/ntsSampler.hpp:857-921), so the batch's hop takes the
largest fanout:
  arxiv     169,343 nodes, 2.48M R-MAT edges, 128 features, fanout [25,10], batch 1,024, 90,941 train nodes
  products  2,449,029 nodes, 126.2M R-MAT edges, 100 features in mapped pinned host memory, HBM cache of the
            top 20 % out-degree nodes, fanout [15,10,5], batch 6,000, 196,615 train nodes
  gat       same graph, fanout [10,10], batch 4,096, 4 heads x 32, fused attention + aggregation fwd+bwd
Everything goes through the C ABI: neighbour sampling of each hop, relabelling, CSR construction,
weights, gathers, aggregation.  --sampler builder (default) builds all layers of a batch in one
stream-ordered sequence with one read-back (nts_batch_builder_*; "sample" then holds sampling and
structure together); --sampler library goes hop by hop through the per-step entry points;
--sampler harness uses the torch sampler of the test harness instead.  Stages are separated by
stream synchronisation, as every reference operator synchronises its stream.  --pipeline 2 samples
the next batch on a second stream while the current one is gathered and aggregated; --pipeline P >= 3
keeps P batches in flight: P - 2 are sampled ahead, each on a stream of its own, and the next
batch's features and labels are gathered on another, so that sampling (small dependent kernels), the
gather (PCIe) and the aggregation (HBM) of consecutive batches overlap; from that depth on the host
does not wait for any aggregation either (--stage-sync 0): batches are ordered by events, and the stage
times printed are host enqueue times.
"""
import argparse
import json
import time

import torch

from . import synth
from .batch import BatchBuilder, FeatureCache, MappedHostTable, load_feature_gpu_cache, load_label_gpu, sample_hop
from .layout import SampledLayer, as_u32
from .ops import GATAggregateOp, GATAttentionOp, SingleGPUSampleGraphOp
from .stream import CudaStream

CONFIGS = {
    "arxiv": dict(V=169_343, E=2_480_000, F=128, hidden=128, classes=40, fanout=[25, 10], batch=1024, train=90_941,
                  seed=2, cache=0.0),
    "products": dict(V=2_449_029, E=126_200_000, F=100, hidden=128, classes=47, fanout=[15, 10, 5], batch=6000,
                     train=196_615, seed=4, cache=0.2),
    "gat": dict(V=2_449_029, E=126_200_000, F=100, hidden=128, classes=47, fanout=[10, 10], batch=4096, train=196_615,
                seed=4, cache=0.2, heads=4),
}


class Timer:
    def __init__(self, sync=True):
        self.t = {}
        self.sync = sync  # False: stages are not waited for, the times are host enqueue times

    def add(self, key, t0):
        # Only the stream the stages run on: a device-wide wait would also wait for the next batch
        # being sampled on the second stream of the pipelined mode.
        if self.sync:
            torch.cuda.current_stream().synchronize()
        self.t[key] = self.t.get(key, 0.0) + time.perf_counter() - t0


def graph_mode(graph, pipeline, cache=0.0):
    """The value for nts_batch_builder_use_graph.  True picks by measurement.  With several batches in
    flight: 1 (one recorded chain of launches; the chains of the other builders already fill the
    chip, extra branches and streams only cost).  With one batch in flight: 3, the transpositions and
    weights as a second graph beside the feature gather (with and without a feature cache: the gather
    keeps no more reads of host memory in flight than the link needs, so the kernels beside it run at
    their usual speed)."""
    if graph is True:
        return 1 if pipeline > 1 else 3
    return int(graph)


def run(name, scale=1.0, max_batches=0, sampler="builder", warmup_batches=2, pipeline=1, quiet=False, checksum=False,
        stage_sync=None, graph=True):
    cfg = dict(CONFIGS[name])
    graph = graph_mode(graph, pipeline, cfg["cache"])
    dev = torch.device("cuda:0")
    V, E = int(cfg["V"] * scale), int(cfg["E"] * scale)
    n_train = int(cfg["train"] * scale)
    src, dst = synth.rmat_edges(V, E, seed=cfg["seed"], device=dev, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    gco, gri = as_u32(co), as_u32(ri)
    out_deg = torch.bincount(src, minlength=V)
    del src, dst
    feat_cpu = synth.normal_features(V, cfg["F"], seed=cfg["seed"] + 40)
    labels = synth.uniform_labels(V, cfg["classes"], seed=cfg["seed"] + 41, device=dev)
    table = MappedHostTable(feat_cpu)
    cache = FeatureCache(feat_cpu, out_deg.cpu(), int(V * cfg["cache"]), dev) if cfg["cache"] > 0 else None
    train_nodes = synth.permutation(V, cfg["seed"] + 42, dev)[:n_train]
    cs = CudaStream()
    # Stages separated by a stream synchronisation, as every reference operator ends with one -- except
    # from three batches in flight on, where the one host thread of this harness would stall all the
    # streams it feeds: there the batches are ordered by events only and the host never waits for an
    # aggregation (the reference gets the same effect from one host thread per pipeline).
    if stage_sync is None:
        stage_sync = not (sampler == "builder" and pipeline > 2)
    tm = Timer(sync=stage_sync)
    heads = cfg.get("heads", 0)
    n_batches = (n_train + cfg["batch"] - 1) // cfg["batch"]
    if max_batches:
        n_batches = min(n_batches, max_batches)
    # graph: a builder records the launches of its hops once and replays them as a HIP graph
    builder = (BatchBuilder(gco, gri, cfg["fanout"], cfg["batch"], want_perm=heads > 0, graph=graph)
               if sampler == "builder" else None)
    train32 = as_u32(train_nodes)
    # pipeline = P > 1 (the reference's PIPELINES mode: P batches in flight, each on a stream of its
    # own and driven by a thread of its own, one batch at a time in each of the sample, transfer and
    # train stages; toolkits/GCN_GPU_NEIGHBOR.hpp:1350-1363 and the stage mutexes of its batch loop).
    # P = 2: the next batch is sampled on a second stream, by a builder of its own, while this one is
    # gathered and aggregated.  P >= 3: P - 2 batches are sampled ahead, each chain of hops on a stream
    # of its own (a chain of small dependent launches gains nothing from a busy chip, several chains
    # side by side do), and the batch after the current one is gathered on a gather stream while the
    # current one aggregates; an event orders each gather before its aggregation.  One host thread
    # enqueues all of it: a producer thread of its own was measured and lost to contention for the
    # interpreter (arxiv 0.039 s against 0.032 s).
    pipelined = builder is not None and pipeline > 1
    staged_gather = pipelined and pipeline > 2
    builders = [builder]
    if pipelined:
        builders += [BatchBuilder(gco, gri, cfg["fanout"], cfg["batch"], want_perm=heads > 0, graph=graph)
                     for _ in range(pipeline - 1)]
        sample_streams = [torch.cuda.Stream(device=dev) for _ in range(max(1, pipeline - 2))]
        gather_stream = torch.cuda.Stream(device=dev) if staged_gather else None
    totals = {"edges": 0, "hits": 0, "rows": 0}
    hits_on_device = torch.zeros(1, dtype=torch.int64, device=dev)  # summed there when no stage is waited for
    checksum_on_device = torch.zeros((), dtype=torch.float64, device=dev)

    def batch_ids(b):
        return train32[b * cfg["batch"]:(b + 1) * cfg["batch"]]

    def gather(stream_obj, layers):
        x = torch.empty(layers[0].src_size, cfg["F"], device=dev)
        if cache is not None:
            hits = load_feature_gpu_cache(stream_obj, layers[0], x, table.dev_ptr, cache)
        else:
            stream_obj.zero_copy_feature_move_gpu(x, table.dev_ptr, layers[0].dev_source, cfg["F"], layers[0].src_size)
            hits = None
        lab = torch.empty(layers[-1].v_size, dtype=torch.int64, device=dev)
        load_label_gpu(stream_obj, layers[-1], lab, labels)
        return x, lab, hits

    def aggregate(layers, x):
        """Forward through the layers (input side first), then backward in reverse order."""
        ops = []
        for l, layer in enumerate(layers):
            width = cfg["F"] if l == 0 else cfg["hidden"]
            if x.shape[1] != width or x.shape[0] != layer.src_size:
                x = synth.normal_features(layer.src_size, width, seed=l, device=dev)  # stands in for the dense layer
            t0 = time.perf_counter()
            if heads:
                H, Fh = heads, cfg["hidden"] // heads
                if x.shape[1] != H * Fh:
                    x = synth.normal_features(layer.src_size, H * Fh, seed=l, device=dev)
                    t0 = time.perf_counter()
                el = x.view(layer.src_size, H, Fh).sum(2).contiguous()
                er = torch.zeros(layer.v_size, H, device=dev)
                att, agg = GATAttentionOp(layer, 0.2), GATAggregateOp(layer, H)
                y = agg.forward(x, att.forward(el, er))
                ops.append((att, agg))
            else:
                op = SingleGPUSampleGraphOp(layers, l, cs, sync=stage_sync)
                y = op.forward(x)
                ops.append(op)
            tm.add("aggregate_fwd", t0)
            x = y
        g = torch.ones_like(x)
        for l in reversed(range(len(layers))):
            if g.shape[0] != layers[l].v_size or g.shape[1] != x.shape[1]:
                g = torch.ones(layers[l].v_size, g.shape[1], device=dev)
            t0 = time.perf_counter()
            if heads:
                att, agg = ops[l]
                g = agg.backward(g)
                att.backward(agg.get_additional_grad())
            else:
                g = ops[l].backward(g)
            tm.add("aggregate_bwd", t0)
        return x, g

    def sample_hop_by_hop(b):
        layers, dst_ids = [], train_nodes[b * cfg["batch"]:(b + 1) * cfg["batch"]]
        for hop, fan in enumerate(cfg["fanout"]):
            t0 = time.perf_counter()
            if sampler == "library":
                dst32 = dst_ids if dst_ids.dtype == torch.int32 else as_u32(dst_ids)
                off32, rows32 = sample_hop(gco, gri, dst32, fan, 1000 * b + hop)
            else:
                d64 = dst_ids.to(torch.int64) & 0xFFFFFFFF
                off, rows_global = synth.sample_hop(co, ri, d64, fan, 1000 * b + hop)
                off32, rows32, dst32 = as_u32(off), as_u32(rows_global), as_u32(d64)
            tm.add("sample", t0)
            t0 = time.perf_counter()
            layer = SampledLayer.from_device_hop(off32, rows32, dst32, V, want_perm=heads > 0)
            tm.add("structure", t0)
            layers.append(layer)
            dst_ids = layer.dev_source
        return layers[::-1]  # input-side layer first

    def finish_batch(layers, x, hits):
        totals["edges"] += sum(l.e_size for l in layers)
        totals["rows"] += layers[0].src_size
        if hits is not None:
            if stage_sync:
                totals["hits"] += int(hits.item())
            else:
                hits_on_device.add_(hits)
        y, g = aggregate(layers, x)
        if checksum:  # of the last layer's output and the first layer's input gradient: equal in every mode
            checksum_on_device.add_(y.double().sum() + g.double().sum())  # no read-back: nothing waits here

    def run_serial(sequence):
        for b in sequence:
            if builder is not None:
                t0 = time.perf_counter()
                builder.enqueue(batch_ids(b), 1000 * b)
                layers = builder.collect(join=False)  # graph mode 3: the transposed structure is still being built
                tm.add("sample", t0)
            else:
                layers = sample_hop_by_hop(b)
            t0 = time.perf_counter()
            x, _, hits = gather(cs, layers)
            tm.add("gather", t0)
            if builder is not None:
                builder.join()  # the aggregation is the first to read the transposed structure and the weights
            finish_batch(layers, x, hits)

    def run_two_stage(sequence):
        if not sequence:
            return

        trained = [None, None]  # per builder: recorded when the batch built in it has been aggregated

        def start_sampling(step):
            # the arena of this builder may still be read by the aggregation of the batch before last
            # (only when the stages are not separated by waits): the sampling stream waits for it
            if trained[step % 2] is not None:
                sample_streams[0].wait_event(trained[step % 2])
            builders[step % 2].enqueue(batch_ids(sequence[step]), 1000 * sequence[step], sample_streams[0].cuda_stream)
        start_sampling(0)
        for step in range(len(sequence)):
            t0 = time.perf_counter()
            layers = builders[step % 2].collect()
            if step + 1 < len(sequence):
                start_sampling(step + 1)
            tm.t["sample_wait"] = tm.t.get("sample_wait", 0.0) + time.perf_counter() - t0
            t0 = time.perf_counter()
            x, _, hits = gather(cs, layers)
            tm.add("gather", t0)
            finish_batch(layers, x, hits)
            trained[step % 2] = torch.cuda.Event()
            trained[step % 2].record(torch.cuda.current_stream())

    def run_staged(sequence):
        if not sequence:
            return
        chains = len(sample_streams)
        started = 0
        trained = [None] * pipeline  # per builder: recorded when the batch built in it has been aggregated

        def sample_through(last_step):
            nonlocal started
            while started <= min(last_step, len(sequence) - 1):
                stream = sample_streams[started % chains]
                if trained[started % pipeline] is not None:
                    stream.wait_event(trained[started % pipeline])  # the arena's last batch is still being read
                builders[started % pipeline].enqueue(batch_ids(sequence[started]), 1000 * sequence[started],
                                                     stream.cuda_stream)
                started += 1

        def start_gather(step):
            """Waits for the sampled layers of `step`, then enqueues the gather of its features and labels."""
            layers = builders[step % pipeline].collect()
            with torch.cuda.stream(gather_stream):
                x, lab, hits = gather(CudaStream(gather_stream.cuda_stream, synchronize=False), layers)
                done = torch.cuda.Event()
                done.record(gather_stream)
            return layers, x, lab, hits, done

        main = torch.cuda.current_stream()
        sample_through(chains - 1)
        staged = start_gather(0)
        sample_through(chains)
        for step in range(len(sequence)):
            # Batch `step` trains below out of builder step % P; batch step + 1 is gathered out of the
            # next builder; the P - 2 after it are being sampled.  Builder (step - 1) % P, whose batch
            # has trained, takes the chain started here.
            t0 = time.perf_counter()
            layers, x, lab, hits, gathered = staged
            if step + 1 < len(sequence):
                staged = start_gather(step + 1)
            sample_through(step + pipeline - 1)
            tm.t["enqueue"] = tm.t.get("enqueue", 0.0) + time.perf_counter() - t0
            t0 = time.perf_counter()
            main.wait_event(gathered)
            for t in (x, lab, hits):
                if t is not None:
                    t.record_stream(main)  # allocated on the gather stream, used on this one
            tm.add("gather_wait", t0)
            finish_batch(layers, x, hits)
            trained[step % pipeline] = torch.cuda.Event()
            trained[step % pipeline].record(main)

    run_batches = run_staged if staged_gather else run_two_stage if pipelined else run_serial
    # The first batches load every kernel's code and grow the allocator's pools; they are run once
    # untimed, as a short epoch of their own (the pipeline drains before the clock starts), then the
    # epoch starts over from its first batch.
    n_warm = min(warmup_batches, n_batches)
    run_batches(list(range(n_warm)))
    torch.cuda.synchronize()
    tm.t.clear()
    totals.update(edges=0, hits=0, rows=0)
    hits_on_device.zero_()
    checksum_on_device.zero_()
    t_epoch = time.perf_counter()
    run_batches(list(range(n_batches)))
    torch.cuda.synchronize()
    epoch_s = time.perf_counter() - t_epoch
    edges_total, hits_total, rows_total = totals["edges"], totals["hits"] + int(hits_on_device.item()), totals["rows"]
    table.close()
    out = {
        "config": name, "scale": scale, "vertices": V, "edges": E, "batches": n_batches, "batch_size": cfg["batch"],
        "warmup_batches": n_warm,
        "fanout_output_side_first": cfg["fanout"], "epoch_s": round(epoch_s, 4),
        "stage_s": {k: round(v, 4) for k, v in tm.t.items()},
        "library_s": round(sum(v for k, v in tm.t.items() if k != "sample" or sampler != "harness"), 4),
        "sampler": sampler, "hop_launches_as_graph": bool(graph and sampler == "builder"),
        "hop_graph_mode": graph if sampler == "builder" else 0,
        "pipeline": pipeline if pipelined else 1, "stage_sync": stage_sync,
        "sampled_edges": edges_total, "gathered_rows": rows_total,
        "cache_hit_rate": round(hits_total / max(rows_total, 1), 4) if cache is not None else None,
        "checksum": float(checksum_on_device.item()) if checksum else None,
    }
    for b in builders:
        if b is not None:
            b.close()
    if not quiet:
        print(json.dumps(out))
    return out


def write_native_inputs(name, directory, scale=1.0, keep_host=False):
    """Writes the arrays of a configuration for lib/nts_epoch: co.bin, ri.bin (uint32 CSC of the whole
    graph), feat.bin (float32 [V, F]), labels.bin (int64 [V]), train.bin (uint32 ids).  Same graph, train
    ids and seeds as `run`.  The products and gat configurations share every file.  Returns the shape
    (and, with keep_host, the host arrays, for a checker)."""
    import os

    cfg = dict(CONFIGS[name])
    dev = torch.device("cuda:0")
    V, E = int(cfg["V"] * scale), int(cfg["E"] * scale)
    n_train = int(cfg["train"] * scale)
    src, dst = synth.rmat_edges(V, E, seed=cfg["seed"], device=dev, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    del src, dst
    host = dict(co=as_u32(co).cpu().numpy(), ri=as_u32(ri).cpu().numpy(),
                feat=synth.normal_features(V, cfg["F"], seed=cfg["seed"] + 40).numpy(),
                labels=synth.uniform_labels(V, cfg["classes"], seed=cfg["seed"] + 41, device=dev).cpu().numpy(),
                train=as_u32(synth.permutation(V, cfg["seed"] + 42, dev)[:n_train]).cpu().numpy())
    del co, ri
    torch.cuda.empty_cache()
    for key, arr in host.items():
        arr.tofile(os.path.join(directory, f"{key}.bin"))
    out = dict(V=V, E=E, n_train=n_train)
    if keep_host:
        import numpy as np

        out.update(co=host["co"].view(np.uint32), ri=host["ri"].view(np.uint32), feat=host["feat"], labels=host["labels"],
                   train=host["train"].view(np.uint32))
    return out


def run_native_on(directory, name, V, max_batches=0, warmup_batches=2, pipeline=1, graph=True, verify=False,
                  stage_sync=False, dump_dir=None, dump_batch=0):
    """Runs lib/nts_epoch on the arrays `write_native_inputs` left in `directory`; returns its JSON line."""
    import os
    import subprocess

    cfg = dict(CONFIGS[name])
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "nts_epoch")
    if not os.path.exists(exe):
        raise RuntimeError(f"{exe} has not been built (make -C neutronbench_amd/csrc)")
    cmd = [exe, "--dir", directory, "--V", str(V), "--F", str(cfg["F"]), "--hidden", str(cfg["hidden"]), "--batch",
           str(cfg["batch"]), "--fanout", ",".join(map(str, cfg["fanout"])), "--heads", str(cfg.get("heads", 0)),
           "--pipeline", str(pipeline), "--cache", str(cfg["cache"]), "--graph",
           str(graph_mode(graph, pipeline, cfg["cache"])), "--warmup", str(warmup_batches), "--max-batches",
           str(max_batches), "--verify", str(int(verify)), "--stage-sync", str(int(stage_sync))]
    if dump_dir:
        cmd += ["--dump-dir", dump_dir, "--dump-batch", str(dump_batch)]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if p.returncode != 0:
        raise RuntimeError(f"nts_epoch failed ({p.returncode}): {p.stderr[-2000:]}")
    return json.loads(p.stdout.strip().splitlines()[-1])


def run_native(name, scale=1.0, max_batches=0, warmup_batches=2, pipeline=1, quiet=False, graph=True, verify=False,
               stage_sync=False, keep_dir=None):
    """The same epoch driven from C++ (neutronbench_amd/host/epoch_driver.cpp -> lib/nts_epoch): the
    arrays of the synthetic configuration are written to a directory, the program runs the batches
    through the C ABI with no Python between the calls and prints one JSON line.  Same graph, train
    ids and seeds as `run`, so sampled_edges and gathered_rows are equal."""
    import shutil
    import tempfile

    cfg = dict(CONFIGS[name])
    d = keep_dir or tempfile.mkdtemp(prefix="nts_epoch_")
    try:
        shape = write_native_inputs(name, d, scale)
        out = run_native_on(d, name, shape["V"], max_batches, warmup_batches, pipeline, graph, verify, stage_sync)
    finally:
        if keep_dir is None:
            shutil.rmtree(d, ignore_errors=True)
    out.update(config=name, scale=scale, vertices=shape["V"], edges=shape["E"], fanout_output_side_first=cfg["fanout"])
    if not quiet:
        print(json.dumps(out))
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", choices=sorted(CONFIGS), required=True)
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--max-batches", type=int, default=0)
    ap.add_argument("--sampler", choices=["builder", "library", "harness"], default="builder")
    ap.add_argument("--warmup-batches", type=int, default=2, help="untimed batches before the epoch starts")
    ap.add_argument("--pipeline", type=int, default=1, choices=[1, 2, 3, 4, 5, 6],
                    help="batches in flight. 2: the next batch is sampled on a second stream while this one is "
                         "gathered and aggregated; 3 and more: P - 2 batches are sampled ahead and the next one is "
                         "gathered on a stream of its own")
    ap.add_argument("--stage-sync", type=int, default=None, choices=[0, 1],
                    help="1: wait for the stream after every stage (stage times are device times; default up to "
                         "--pipeline 2); 0: never wait for an aggregation, batches are ordered by events (stage times "
                         "are host enqueue times; default from --pipeline 3)")
    ap.add_argument("--graph", type=int, default=None, choices=[0, 1, 2, 3],
                    help="1: each builder replays the launches of its hops as a HIP graph recorded at its first "
                         "batch; 2: the same with each hop's transposition and weights on a side branch of the graph; "
                         "3: transpositions and weights as a second graph on the builder's own stream, beside the "
                         "gather; 0: the launches are enqueued one by one for every batch; default for --pipeline 1: "
                         "3 with a feature cache, 2 without; else 1")
    ap.add_argument("--native", action="store_true",
                    help="drive the epoch from C++ (lib/nts_epoch) instead of this module's Python loop")
    ap.add_argument("--write-inputs", metavar="DIR", default=None,
                    help="only write the configuration's arrays for lib/nts_epoch to DIR and print the command line "
                         "that runs the epoch on them (to run the program under a profiler)")
    a = ap.parse_args()
    if a.write_inputs:
        import os

        os.makedirs(a.write_inputs, exist_ok=True)
        shape = write_native_inputs(a.config, a.write_inputs, a.scale)
        cfg = CONFIGS[a.config]
        print(" ".join(["neutronbench_amd/lib/nts_epoch", "--dir", a.write_inputs, "--V", str(shape["V"]), "--F",
                        str(cfg["F"]), "--hidden", str(cfg["hidden"]), "--batch", str(cfg["batch"]), "--fanout",
                        ",".join(map(str, cfg["fanout"])), "--heads", str(cfg.get("heads", 0)), "--cache",
                        str(cfg["cache"]), "--pipeline", str(a.pipeline), "--stage-sync",
                        str(int(bool(a.stage_sync)) if a.stage_sync is not None else 1), "--graph",
                        str(graph_mode(True if a.graph is None else a.graph, a.pipeline, cfg["cache"]))]))
    elif a.native:
        run_native(a.config, a.scale, a.max_batches, a.warmup_batches, a.pipeline,
                   graph=True if a.graph is None else a.graph, stage_sync=bool(a.stage_sync))
    else:
        run(a.config, a.scale, a.max_batches, a.sampler, a.warmup_batches, a.pipeline,
            stage_sync=None if a.stage_sync is None else bool(a.stage_sync),
            graph=True if a.graph is None else a.graph)
