"""Whole-batch construction on the device (nts_batch_builder_*) against the per-hop entry points and
the CPU oracle: every array of every layer, bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import host_u32
from neutronbench_amd import abi, synth
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.batch import BatchBuilder, sample_hop
from neutronbench_amd.layout import SampledLayer, as_u32

pytestmark = pytest.mark.gpu


def graph(V, E, seed, device):
    src, dst = synth.rmat_edges(V, E, seed=seed, device=device, sort=True)
    co, ri = synth.build_csc(src, dst, V)
    return as_u32(co), as_u32(ri)


def per_hop_layers(gco, gri, batch, fanouts, seed, V):
    """The same batch through the per-hop entry points (a read-back after every step)."""
    layers, dst = [], batch
    for h, fan in enumerate(fanouts):
        co, ri = sample_hop(gco, gri, dst, fan, seed + h)
        layers.append(SampledLayer.from_device_hop(co, ri, dst, V, want_perm=True))
        dst = layers[-1].dev_source
    return layers[::-1]


ARRAYS = ("dev_destination", "dev_source", "dev_column_offset", "dev_row_indices", "dev_row_offset",
          "dev_column_indices", "dev_csr_to_csc", "dev_edge_weight_forward", "dev_edge_weight_backward")


def assert_same_layers(got, want):
    assert len(got) == len(want)
    for k, (a, b) in enumerate(zip(got, want)):
        assert (a.v_size, a.e_size, a.src_size) == (b.v_size, b.e_size, b.src_size), f"layer {k}"
        for name in ARRAYS:
            x, y = getattr(a, name), getattr(b, name)
            assert x.numel() == y.numel(), f"layer {k} {name}"
            assert x.cpu().numpy().tobytes() == y.cpu().numpy().tobytes(), f"layer {k} {name}"


@pytest.mark.parametrize("V,E,batch,fanouts,seed", [
    (30000, 600000, 1024, [25, 10], 1),          # the Arxiv-shaped configuration's hops
    (50000, 2000000, 3000, [15, 10, 5], 2),      # Products-shaped hops
    (4000, 30000, 500, [3, 2, 2, 2], 3),         # more hops than layers of the configurations, sparse graph
    (2000, 400000, 64, [64, 100], 4),            # fanout of a whole wavefront and the permutation pick above it
    (3000, 40000, 700, [-1, 4], 5),              # whole neighbourhoods first
])
def test_builder_equals_the_per_hop_entry_points(device, V, E, batch, fanouts, seed):
    gco, gri = graph(V, E, seed, device)
    ids = as_u32(synth.permutation(V, seed + 10, device)[:batch])
    builder = BatchBuilder(gco, gri, fanouts, batch, want_perm=True)
    got = builder.sample(ids, 1000 * seed)
    want = per_hop_layers(gco, gri, ids, fanouts, 1000 * seed, V)
    assert_same_layers(got, want)
    assert got[-1].dev_destination.cpu().numpy().tobytes() == ids.cpu().numpy().tobytes()
    builder.close()


def test_builder_layers_equal_the_oracle_construction(device):
    """Directly against the restated host algorithms (postprocessing, generate_csr_from_csc,
    update_degree + compute_weight_*) on the sampled lists the builder picked."""
    V, E, batch, fanouts = 20000, 500000, 800, [6, 12]
    gco, gri = graph(V, E, 21, device)
    ids = as_u32(synth.permutation(V, 22, device)[:batch])
    builder = BatchBuilder(gco, gri, fanouts, batch)
    layers = builder.sample(ids, 5)
    gco_h, gri_h = host_u32(gco), host_u32(gri)
    dst = host_u32(ids)
    for hop, layer in enumerate(layers[::-1]):
        co = host_u32(layer.dev_column_offset)
        assert np.array_equal(co, oracle.init_co(gco_h, dst, fanouts[hop]))
        local, source = host_u32(layer.dev_row_indices), host_u32(layer.dev_source)
        glob = source[local]
        for i in range(0, dst.size, 37):  # sampled sources are in-neighbours of their destination
            seg = gri_h[gco_h[dst[i]]:gco_h[dst[i] + 1]]
            assert np.isin(glob[co[i]:co[i + 1]], seg).all()
        want_local, want_source, n = oracle.postprocess(glob, V)
        assert n == layer.src_size and np.array_equal(source, want_source) and np.array_equal(local, want_local)
        ro, ci = oracle.csr_from_csc(co, local, n)
        assert np.array_equal(host_u32(layer.dev_row_offset), ro)
        assert np.array_equal(host_u32(layer.dev_column_indices), ci)
        outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
        ewf, ewb = oracle.layer_weights(co, local, ro, ci, source, dst, outd, ind)
        assert layer.dev_ewf().cpu().numpy().tobytes() == ewf.tobytes()
        assert layer.dev_ewb().cpu().numpy().tobytes() == ewb.tobytes()
        assert layer.dev_csr_to_csc is None
        dst = source
    builder.close()


def test_builder_reused_over_batches_of_changing_size(device):
    """One builder, batches large -> tiny -> empty -> one vertex -> large: nothing of an earlier
    batch shows in a later one (the arena keeps stale data beyond the live counts)."""
    V, E, fanouts = 20000, 300000, [8, 8]
    gco, gri = graph(V, E, 31, device)
    # a few isolated vertices: no in-edges
    deg = host_u32(gco)[1:] - host_u32(gco)[:-1]
    isolated = np.nonzero(deg == 0)[0][:5]
    perm = synth.permutation(V, 32, device)
    builder = BatchBuilder(gco, gri, fanouts, 2048, want_perm=True)
    batches = [perm[:2048], perm[100:103], perm[:0], perm[7:8], perm[2048:4096]]
    if isolated.size:
        batches.insert(2, torch.from_numpy(isolated.astype(np.int64)).to(device))
    for k, ids64 in enumerate(batches):
        ids = as_u32(ids64)
        got = builder.sample(ids, 40 + k)
        if ids.numel() == 0:
            assert all((l.v_size, l.e_size, l.src_size) == (0, 0, 0) for l in got)
            assert all(host_u32(l.dev_column_offset).tolist() == [0] and host_u32(l.dev_row_offset).tolist() == [0]
                       for l in got)
            continue
        want = per_hop_layers(gco, gri, ids, fanouts, 40 + k, V)
        assert_same_layers(got, want)
    builder.close()


def test_builder_rejects_what_it_cannot_hold(device):
    gco, gri = graph(1000, 8000, 41, device)
    V, E = 1000, 8000
    fan = (ctypes.c_int32 * 2)(4, 4)
    assert call("nts_batch_builder_arena_bytes", V, E, fan, 0, 16, 0) == 0
    assert call("nts_batch_builder_arena_bytes", V, E, fan, 9, 16, 0) == 0
    assert call("nts_batch_builder_arena_bytes", V, E, fan, 2, 0, 0) == 0
    need = call("nts_batch_builder_arena_bytes", V, E, fan, 2, 16, 0)
    arena = torch.empty(need + 256, dtype=torch.uint8, device=device)
    base = (arena.data_ptr() + 255) // 256 * 256
    handle = ctypes.c_void_p()
    args = (ptr(gco), ptr(gri), V, E, fan, 2, 16, 0)
    assert abi.status("nts_batch_builder_create", ctypes.byref(handle), *args, base, need - 1) == abi.NTS_ERR_INVALID
    assert "arena" in abi.last_error()
    assert abi.status("nts_batch_builder_create", ctypes.byref(handle), *args, base + 4, need) == abi.NTS_ERR_INVALID
    zero = (ctypes.c_int32 * 2)(4, 0)
    assert abi.status("nts_batch_builder_create", ctypes.byref(handle), ptr(gco), ptr(gri), V, E, zero, 2, 16, 0, base,
                      need) == abi.NTS_ERR_INVALID
    call("nts_batch_builder_create", ctypes.byref(handle), *args, base, need)
    desc = (abi.SampledLayerDesc * 2)()
    assert abi.status("nts_batch_builder_layers", handle.value, ctypes.addressof(desc)) == abi.NTS_ERR_INVALID
    ids = torch.arange(17, dtype=torch.int32, device=device)
    s = torch.cuda.current_stream().cuda_stream
    assert abi.status("nts_batch_builder_sample", handle.value, ptr(ids), 17, 1, s) == abi.NTS_ERR_INVALID
    assert "max_batch" in abi.last_error()
    call("nts_batch_builder_sample", handle.value, ptr(ids), 16, 1, s)
    call("nts_batch_builder_layers", handle.value, ctypes.addressof(desc))
    assert desc[1].v_size == 16 and desc[0].v_size == desc[1].src_size
    call("nts_batch_builder_destroy", handle.value)


def test_two_builders_on_two_streams_overlap_without_interference(device):
    """The pipelined use: batch k+1 is built by a second builder on a second stream while batch k's
    layers are still being read.  Each batch equals what a lone builder gives for it."""
    V, E, fanouts, batch = 40000, 900000, [10, 15], 2000
    gco, gri = graph(V, E, 51, device)
    perm = as_u32(synth.permutation(V, 52, device))
    lone = BatchBuilder(gco, gri, fanouts, batch, want_perm=True)
    want = []
    for k in range(6):
        layers = lone.sample(perm[k * batch:(k + 1) * batch], 90 + k)
        want.append([{name: getattr(l, name).cpu().numpy().copy() for name in ARRAYS} for l in layers])
    lone.close()
    builders = [BatchBuilder(gco, gri, fanouts, batch, want_perm=True) for _ in range(2)]
    streams = [torch.cuda.Stream(device=device) for _ in range(2)]
    torch.cuda.synchronize()
    builders[0].enqueue(perm[0:batch], 90, streams[0].cuda_stream)
    for k in range(6):
        if k + 1 < 6:  # start the next batch before this one is collected
            builders[(k + 1) % 2].enqueue(perm[(k + 1) * batch:(k + 2) * batch], 91 + k, streams[(k + 1) % 2].cuda_stream)
        layers = builders[k % 2].collect()
        for l, expect in zip(layers, want[k]):
            for name in ARRAYS:
                assert getattr(l, name).cpu().numpy().tobytes() == expect[name].tobytes(), f"batch {k} {name}"
    for b in builders:
        b.close()


@pytest.mark.parametrize("mode", [1, 2, 3])
@pytest.mark.parametrize("fanouts,want_perm", [([25, 10], True), ([15, 10, 5], True), ([64, 100], True)])
def test_builder_replaying_a_graph_equals_the_launch_by_launch_builder(device, fanouts, want_perm, mode):
    """nts_batch_builder_use_graph: the hops' launches are recorded at the first batch and replayed
    for every later one (mode 1: as one chain; mode 2: each hop's transposition and weights on a
    side branch of the graph, beside the next hop's sampling; mode 3: the transpositions and weights
    as a second graph on a stream of the builder's, which `sample` joins to the current stream).  Replays are interleaved with eager work and synchronisations of the
    program's own (the per-hop path run for comparison, read-backs), batch sizes and seeds change
    from replay to replay, and every replay must give the arrays of the eager builder bit for bit."""
    V, E, cap = 30000, 700000, 1500
    gco, gri = graph(V, E, 61, device)
    perm = synth.permutation(V, 62, device)
    eager = BatchBuilder(gco, gri, fanouts, cap, want_perm=want_perm)
    replay = BatchBuilder(gco, gri, fanouts, cap, want_perm=want_perm, graph=mode)
    sizes = [1500, 1500, 640, 1, 0, 1499, 77, 1500]
    at = 0
    for k, n in enumerate(sizes):
        ids = as_u32(perm[at:at + n])
        at += n
        got = replay.sample(ids, 7000 + 13 * k)
        want = eager.sample(ids, 7000 + 13 * k)
        assert_same_layers(got, want)
        if n and k % 3 == 0:  # and both equal the per-hop entry points
            assert_same_layers(got, per_hop_layers(gco, gri, ids, fanouts, 7000 + 13 * k, V))
        torch.cuda.synchronize()
    eager.close()
    replay.close()


def test_graph_builders_on_two_streams(device):
    """Two builders in graph mode, each captured on and replayed to a stream of its own while the
    other one's batch is still in flight."""
    V, E, fanouts, batch = 40000, 900000, [10, 15], 2000
    gco, gri = graph(V, E, 71, device)
    perm = as_u32(synth.permutation(V, 72, device))
    lone = BatchBuilder(gco, gri, fanouts, batch, want_perm=True)
    want = []
    for k in range(6):
        layers = lone.sample(perm[k * batch:(k + 1) * batch], 190 + k)
        want.append([{name: getattr(l, name).cpu().numpy().copy() for name in ARRAYS} for l in layers])
    lone.close()
    builders = [BatchBuilder(gco, gri, fanouts, batch, want_perm=True, graph=True) for _ in range(2)]
    streams = [torch.cuda.Stream(device=device) for _ in range(2)]
    torch.cuda.synchronize()
    builders[0].enqueue(perm[0:batch], 190, streams[0].cuda_stream)
    for k in range(6):
        if k + 1 < 6:
            builders[(k + 1) % 2].enqueue(perm[(k + 1) * batch:(k + 2) * batch], 191 + k, streams[(k + 1) % 2].cuda_stream)
        layers = builders[k % 2].collect()
        for l, expect in zip(layers, want[k]):
            for name in ARRAYS:
                assert getattr(l, name).cpu().numpy().tobytes() == expect[name].tobytes(), f"batch {k} {name}"
    for b in builders:
        b.close()


def test_deferred_structure_is_joined_by_the_stream_that_reads_it(device):
    """Graph mode 3: nts_batch_builder_layers returns when the sampled half of the batch is complete
    (ids, offsets, local row indices: readable at once from any stream) while the transposed structure
    and the weights are still being built on the builder's own stream; a stream that reads those calls
    nts_batch_builder_join first.  The next batch is enqueued without any wait for that second half
    from the caller (the builder orders it); every array equals the launch-by-launch builder's."""
    V, E, fanouts, cap = 40000, 900000, [12, 9, 6], 1200
    gco, gri = graph(V, E, 81, device)
    perm = as_u32(synth.permutation(V, 82, device))
    eager = BatchBuilder(gco, gri, fanouts, cap, want_perm=True)
    deferred = BatchBuilder(gco, gri, fanouts, cap, want_perm=True, graph=3)
    sampled_half = ("dev_destination", "dev_source", "dev_column_offset", "dev_row_indices")
    producer, reader = torch.cuda.Stream(device=device), torch.cuda.Stream(device=device)
    at = 0
    for k, n in enumerate([1200, 1200, 500, 0, 1199, 3, 1200]):
        ids = perm[at:at + n]
        at += n
        want = eager.sample(ids, 300 + k)
        torch.cuda.synchronize()
        deferred.enqueue(ids, 300 + k, producer.cuda_stream)
        layers = deferred.collect(join=False)
        with torch.cuda.stream(reader):
            first = [{name: getattr(l, name).tensor().clone() for name in sampled_half} for l in layers]
            deferred.join(reader.cuda_stream)
            rest = [{name: getattr(l, name).tensor().clone() for name in ARRAYS if name not in sampled_half}
                    for l in layers]
        reader.synchronize()
        for l, a, b in zip(want, first, rest):
            for name, got in {**a, **b}.items():
                assert torch.equal(got, getattr(l, name).tensor()), f"batch {k} {name}"
    eager.close()
    deferred.close()
