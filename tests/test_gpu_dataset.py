"""Edge list -> device CSC / CSR / weights (nts_chunk_from_edges) against the oracle's
PartitionToChunks restatement, and the dataset files end to end: .edge and text files on disk ->
pinned tables -> device structures -> zero-copy gather and aggregation."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host_u32
from neutronbench_amd import dataset, synth
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.layout import FullGraphChunk
from neutronbench_amd.ops import ForwardSingleGPUfuseOp
from neutronbench_amd.stream import CudaStream
from util import abs_term_scale, check

pytestmark = pytest.mark.gpu


def reference_chunk(src, dst, V):
    """The oracle's chunk for an edge list in file order: the reference lists edges by source, and
    within a source in the order its loader appended them, which for one thread is the file order."""
    order = np.argsort(src, kind="stable")
    coo_s, coo_d = src[order].astype(np.uint32), dst[order].astype(np.uint32)
    outd, ind = oracle.degrees(coo_s, coo_d, V)
    return oracle.build_chunk(coo_s, coo_d, V, outd, ind)


def assert_chunk_equals(chunk, ref):
    for name, t in (("co", chunk.column_offset_gpu), ("ri", chunk.row_indices_gpu), ("ro", chunk.row_offset_gpu),
                    ("ci", chunk.column_indices_gpu)):
        assert np.array_equal(host_u32(t), ref[name]), name
    assert chunk.edge_weight_forward_gpu.cpu().numpy().tobytes() == ref["ewf"].tobytes()
    assert chunk.edge_weight_backward_gpu.cpu().numpy().tobytes() == ref["ewb"].tobytes()


@pytest.mark.parametrize("V,E,seed", [(1, 5, 0), (7, 40, 1), (1000, 20000, 2), (5000, 300000, 3), (70000, 100000, 4)])
def test_chunk_from_edges_matches_oracle(device, V, E, seed):
    rng = np.random.default_rng(seed)
    # skewed ids: duplicates, self loops and vertices without edges all occur
    src = np.minimum((rng.random(E) ** 2 * V).astype(np.int64), V - 1)
    dst = np.minimum((rng.random(E) ** 3 * V).astype(np.int64), V - 1)
    pairs = dev(np.stack([src, dst], 1).astype(np.int32), device)
    chunk = FullGraphChunk.from_edge_pairs(pairs, V)
    assert_chunk_equals(chunk, reference_chunk(src, dst, V))


def test_chunk_from_edges_without_edges_or_weights(device):
    V = 33
    co = torch.full((V + 1,), -1, dtype=torch.int32, device=device)
    ro = torch.full((V + 1,), -1, dtype=torch.int32, device=device)
    call("nts_chunk_from_edges", ptr(co), 0, 0, ptr(ro), 0, 0, 0, 0, V, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert not co.any() and not ro.any()
    # structure only (both weight pointers NULL)
    rng = np.random.default_rng(9)
    src, dst = rng.integers(0, V, 500), rng.integers(0, V, 500)
    pairs = dev(np.stack([src, dst], 1).astype(np.int32), device)
    ri = torch.empty(500, dtype=torch.int32, device=device)
    ci = torch.empty(500, dtype=torch.int32, device=device)
    work = torch.empty(call("nts_chunk_from_edges_work_bytes", V, 500) + 256, dtype=torch.uint8, device=device)
    call("nts_chunk_from_edges", ptr(co), ptr(ri), 0, ptr(ro), ptr(ci), 0, ptr(pairs), 500, V,
         (work.data_ptr() + 255) // 256 * 256, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    ref = reference_chunk(src, dst, V)
    assert np.array_equal(host_u32(co), ref["co"]) and np.array_equal(host_u32(ri), ref["ri"])
    assert np.array_equal(host_u32(ro), ref["ro"]) and np.array_equal(host_u32(ci), ref["ci"])


def test_dataset_files_end_to_end(device, tmp_path):
    """Files in the generator's formats -> GNNDatum tables in mapped pinned memory + device chunk ->
    zero-copy row gather and aggregation, all against the oracle fed by its own readers."""
    rng = np.random.default_rng(21)
    V, E, F = 3000, 40000, 24
    src, dst = synth.rmat_edges(V, E, seed=5)
    pairs = np.stack([src.numpy(), dst.numpy()], 1).astype(np.uint32)
    dataset.write_edge_file(tmp_path / "g.edge", pairs)
    x = rng.standard_normal((V, F)).astype(np.float32)
    labels = rng.integers(0, 40, V)
    with open(tmp_path / "g.feat", "w") as f:
        for i, r in enumerate(x):
            f.write(str(i) + " " + " ".join("%.4f" % v for v in r) + "\n")
    with open(tmp_path / "g.label", "w") as f, open(tmp_path / "g.mask", "w") as m:
        for i in range(V):
            f.write(f"{i} {labels[i]}\n")
            m.write(f"{i} {('train', 'val', 'test')[i % 3]}\n")

    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", V, F)
    osrc, odst = oracle.read_edges(tmp_path / "g.edge")
    ref = reference_chunk(osrc.astype(np.int64), odst.astype(np.int64), V)

    datum = dataset.GNNDatum(V, F, pinned=True)
    datum.readFeature_Label_Mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask")
    assert np.array_equal(datum.local_feature.view(np.uint32), o["local_feature"].view(np.uint32))
    assert np.array_equal(datum.local_label, o["local_label"]) and np.array_equal(datum.local_mask, o["local_mask"])
    chunk = FullGraphChunk.from_edge_file(tmp_path / "g.edge", V, device)
    assert_chunk_equals(chunk, ref)

    # zero-copy gather of sampled rows from the pinned table the reader filled
    ids = rng.integers(0, V, 777).astype(np.uint32)
    out = torch.empty((777, F), dtype=torch.float32, device=device)
    cs = CudaStream(torch.cuda.current_stream().cuda_stream)
    cs.zero_copy_feature_move_gpu(out, datum.dev_local_feature, dev(ids.view(np.int32), device), F, 777)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.get_feature(o["local_feature"], ids).view(np.uint32))

    # aggregation over the loaded graph on the loaded features
    feat = o["local_feature"]
    y = ForwardSingleGPUfuseOp(chunk).forward(dev(feat, device)).cpu().numpy()
    check(y, oracle.spmm(feat, ref["ewf"], ref["co"], ref["ri"], V),
          abs_term_scale(feat, ref["ewf"], ref["co"], ref["ri"], V))

    # the binary table holds the same bits and needs no parsing
    datum.write_feature_table(tmp_path / "g.featbin")
    again = dataset.GNNDatum(V, F, pinned=True)
    again.read_feature_table(tmp_path / "g.featbin")
    assert np.array_equal(again.local_feature.view(np.uint32), o["local_feature"].view(np.uint32))
    datum.close()
    again.close()


def test_chunk_from_edges_full_size_properties(device):
    """Reddit-shaped list (114.8 M edges): structure checked through properties that do not need the
    sequential oracle -- against a stable two-key sort done with torch, offsets as histograms, and
    the weight identity between the two orders."""
    V, E = 232965, 114_800_000
    src, dst = synth.rmat_edges(V, E, seed=3, device=device)
    chunk = FullGraphChunk.from_edges(src, dst, V)
    co, ro = chunk.column_offset_gpu.to(torch.int64), chunk.row_offset_gpu.to(torch.int64)
    assert torch.equal(co[1:] - co[:-1], torch.bincount(dst, minlength=V))
    assert torch.equal(ro[1:] - ro[:-1], torch.bincount(src, minlength=V))
    assert int(co[0]) == 0 and int(co[-1]) == E and int(ro[0]) == 0 and int(ro[-1]) == E
    order = torch.sort(src, stable=True).indices
    coo_dst = dst[order]
    assert torch.equal(chunk.column_indices_gpu.to(torch.int64), coo_dst)
    coo_src = src[order]
    del order
    perm = torch.sort(coo_dst, stable=True).indices
    assert torch.equal(chunk.row_indices_gpu.to(torch.int64), coo_src[perm])
    # the k-th CSR edge and its CSC position carry the same weight
    assert torch.equal(chunk.edge_weight_forward_gpu, chunk.edge_weight_backward_gpu[perm])
    # spot check of the weight formula on a sample of edges
    idx = torch.randint(0, E, (4096,), device=device)
    ri = chunk.row_indices_gpu.to(torch.int64)[idx].cpu().numpy()
    d_of = (torch.searchsorted(co, idx, right=True) - 1).cpu().numpy()
    outd = (ro[1:] - ro[:-1]).cpu().numpy()
    ind = (co[1:] - co[:-1]).cpu().numpy()
    want = np.array([oracle.norm_degree(int(outd[s]), int(ind[d])) for s, d in zip(ri, d_of)], dtype=np.float32)
    assert chunk.edge_weight_forward_gpu[idx].cpu().numpy().tobytes() == want.tobytes()


@pytest.mark.parametrize("classes,fmt,sep,shuffled", [(1, "%.4f", " ", False), (1, "%.9g", "\t", True),
                                                      (12, "%.6e", " ", True)])
def test_readers_match_the_reference_data_loader(device, tmp_path, classes, fmt, sep, shuffled):
    """The reference's own GNNDatum::readFeature_Label_Mask (built from its tree, run as a program)
    on the same files: the library's reader and the oracle's restatement give the same five tables
    bit for bit."""
    import refops

    if not refops.available("gpu"):
        pytest.skip("reference-built program not present")
    rng = np.random.default_rng(31 + classes)
    V, F = 1500, 23
    prefix = str(tmp_path / "d")
    np.stack([rng.integers(0, V, 4000), rng.integers(0, V, 4000)], 1).astype(np.uint32).tofile(prefix + ".edge")
    ids = rng.permutation(V) if shuffled else np.arange(V)
    x = (rng.standard_normal((V, F)) * 10.0 ** rng.integers(-3, 4, (V, 1))).astype(np.float32)
    with open(prefix + ".feat", "w") as f:
        for i in ids:
            f.write(str(int(i)) + sep + sep.join(fmt % v for v in x[i]) + "\n")
    with open(prefix + ".label", "w") as f:
        for i in ids:
            if classes > 1:
                idx = rng.choice(classes, rng.integers(0, 4), replace=False)
                f.write(f"{i} {len(idx)} " + " ".join(map(str, idx)) + "\n")
            else:
                f.write(f"{i} {rng.integers(0, 40)}\n")
    words = rng.choice(["train", "val", "eval", "test", "other"], V)
    with open(prefix + ".mask", "w") as f:
        for i in ids:
            f.write(f"{i} {words[i]}\n")
    ref = refops.run_data_loader(V, F, classes, prefix)
    o = oracle.read_feature_label_mask(prefix + ".feat", prefix + ".label", prefix + ".mask", V, F, classes)
    lib = dataset.GNNDatum(V, F, classes, pinned=True)
    lib.readFeature_Label_Mask(prefix + ".feat", prefix + ".label", prefix + ".mask")
    assert np.array_equal(ref["local_feature"].view(np.uint32), o["local_feature"].view(np.uint32))
    assert np.array_equal(ref["local_feature"].view(np.uint32), lib.local_feature.view(np.uint32))
    for k in ("local_label", "global_label", "local_mask", "global_mask"):
        assert np.array_equal(ref[k], o[k]), k
        assert np.array_equal(ref[k], getattr(lib, k)), k
    lib.close()
