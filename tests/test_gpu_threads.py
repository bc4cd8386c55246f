"""Two host threads drive the library at the same time, each on a stream of its own (the reference
runs one host thread per pipeline, toolkits/GCN_GPU_NEIGHBOR.hpp:1350-1363).  The entry points used
here take scratch from the library's per-device pool, keep per-thread caches and report errors per
thread; every result must equal, bit for bit, what one thread computes alone."""
import threading

import numpy as np
import pytest
import torch

from gpu_util import dev
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.batch import MappedHostTable

pytestmark = pytest.mark.gpu


def _graph(seed, Vd=20000, Vs=6000):
    rng = np.random.default_rng(seed)
    deg = rng.poisson(4, Vd).astype(np.int64)
    deg[5], deg[77] = 30000, 2500            # hub rows: cut on the device, listed as long rows
    co = np.concatenate([[0], np.cumsum(deg)]).astype(np.uint32)
    ri = rng.integers(0, Vs, int(co[-1])).astype(np.uint32)
    return co, ri, Vd, Vs


def _run(device, stream, co, ri, Vd, Vs, x, w, scores, msg, table_ptr, ids, rounds):
    """One worker's sequence of calls on `stream`; returns the last round's outputs."""
    s = stream.cuda_stream
    E, F, H = ri.numel(), x.shape[1], scores.shape[1]
    with torch.cuda.stream(stream):
        out = torch.empty(Vd, F, device=device)
        alpha = torch.empty(E, H, device=device)
        sums = torch.empty(Vd, msg.shape[1], device=device)
        rows = torch.empty(ids.numel(), F, device=device)
        for _ in range(rounds):
            call("nts_spmm_gather", ptr(x), ptr(out), ptr(w), ptr(co), ptr(ri), 0, Vd, E, F, 0, s)
            call("nts_edge_softmax_fwd", ptr(alpha), ptr(scores), ptr(co), Vd, H, s)
            call("nts_gather_edge_to_dst", ptr(sums), ptr(msg), ptr(co), Vd, msg.shape[1], 0, s)
            call("nts_gather_rows_f32", ptr(rows), table_ptr, ptr(ids), 0, 0, ids.numel(), F, s)
        stream.synchronize()
    return out, alpha, sums, rows


def test_two_host_threads_on_two_streams(device):
    work = []
    for seed in (1, 2):
        co, ri, Vd, Vs = _graph(seed)
        rng = np.random.default_rng(10 + seed)
        E = ri.size
        feat = rng.standard_normal((Vs, 64)).astype(np.float32)
        table = MappedHostTable(torch.from_numpy(feat))
        args = dict(co=dev(co, device), ri=dev(ri, device), Vd=Vd, Vs=Vs, x=dev(feat, device),
                    w=dev(rng.random(E).astype(np.float32), device),
                    scores=dev(rng.standard_normal((E, 4)).astype(np.float32), device),
                    msg=dev(rng.standard_normal((E, 8)).astype(np.float32), device), table_ptr=table.dev_ptr,
                    ids=dev(rng.integers(0, Vs, 5000).astype(np.uint32), device))
        work.append((args, table))
    alone = [_run(device, torch.cuda.Stream(device=device), rounds=1, **args) for args, _ in work]
    together = [None, None]
    failures = []

    def worker(k):
        try:
            together[k] = _run(device, torch.cuda.Stream(device=device), rounds=25, **work[k][0])
        except BaseException as exc:  # reported by the main thread
            failures.append(exc)

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures
    for k in range(2):
        for got, want in zip(together[k], alone[k]):
            assert torch.equal(got, want)
    for _, table in work:
        table.close()


def test_two_host_threads_each_replaying_a_builder_graph(device):
    """Two host threads, each with a batch builder of its own in graph mode on a stream of its own: the
    graphs are recorded (thread-local capture) and replayed while the other thread does the same.  Every
    batch equals what a launch-by-launch builder gives alone."""
    from neutronbench_amd import synth
    from neutronbench_amd.batch import BatchBuilder
    from neutronbench_amd.layout import as_u32

    V, E, fanouts, batch, n_batches = 30000, 600000, [12, 8], 1000, 12
    src, dst = synth.rmat_edges(V, E, seed=91, device=device, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    gco, gri = as_u32(co), as_u32(ri)
    names = ("dev_source", "dev_column_offset", "dev_row_indices", "dev_row_offset", "dev_column_indices",
             "dev_edge_weight_forward", "dev_edge_weight_backward")
    perms = [as_u32(synth.permutation(V, 92 + k, device)) for k in range(2)]

    def batches(builder, k, stream):
        out = []
        for b in range(n_batches):
            ids = perms[k][b * batch:(b + 1) * batch - 7 * b]  # shrinking batches
            builder.enqueue(ids, 500 * k + b, stream)
            layers = builder.collect()
            out.append([{n: getattr(l, n).cpu().numpy().copy() for n in names} for l in layers])
        return out

    s0 = torch.cuda.current_stream(device).cuda_stream
    want = []
    for k in range(2):
        plain = BatchBuilder(gco, gri, fanouts, batch)
        want.append(batches(plain, k, s0))
        plain.close()
    got, failures = [None, None], []

    def worker(k):
        try:
            stream = torch.cuda.Stream(device=device)
            builder = BatchBuilder(gco, gri, fanouts, batch, graph=True)
            got[k] = batches(builder, k, stream.cuda_stream)
            builder.close()
        except BaseException as exc:
            failures.append(exc)

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures
    for k in range(2):
        for b in range(n_batches):
            for lg, lw in zip(got[k][b], want[k][b]):
                for n in names:
                    assert lg[n].tobytes() == lw[n].tobytes(), f"thread {k} batch {b} {n}"
