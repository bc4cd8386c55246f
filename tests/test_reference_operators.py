"""The oracle against the REFERENCE'S OWN CPU operators, and the reference's own GPU operator
classes running over libntship against its CPU operators.

oracle/_ref/ref_fullgraph_cpu and ref_fullgraph_gpu are built by oracle/build_ref.sh from the
reference tree (loader, partitioner, ForwardCPUfuseOp, SingleCPUSrcDstScatterOp, SingleEdgeSoftMax,
SingleCPUDstAggregateOp; with CUDA_ENABLE=1 also ForwardSingleGPUfuseOp and the DistGPU* edge
operators, compiled against the HIP veneer).  The tests skip where the programs were not built."""
import numpy as np
import pytest

import oracle
import refops
from util import abs_term_scale, check, planless_piece_edges

CASES = [(300, 4000, 19, 4, 1), (2000, 60000, 64, 1, 2), (5000, 40000, 7, 3, 3)]


def oracle_chunk(inp):
    V = inp["x"].shape[0]
    order = np.argsort(inp["src"], kind="stable")
    cs, cd = inp["src"][order], inp["dst"][order]
    od, idg = oracle.degrees(cs, cd, V)
    return oracle.build_chunk(cs, cd, V, od, idg)


def rows_as_sorted_pairs(offsets, indices, weights):
    """(index, weight bits) pairs sorted inside every row: the row's multiset of edges."""
    keys = np.repeat(np.arange(offsets.size - 1, dtype=np.int64), np.diff(offsets.astype(np.int64)))
    order = np.lexsort((weights.view(np.uint32), indices, keys))
    return indices[order], weights.view(np.uint32)[order]


@pytest.mark.skipif(not refops.available("cpu"), reason="reference-built CPU operator program not present")
@pytest.mark.parametrize("V,E,F,H,seed", CASES)
def test_oracle_matches_the_reference_cpu_operators(tmp_path, V, E, F, H, seed):
    inp = refops.make_inputs(V, E, F, H, seed)
    ref = refops.run("cpu", "cpu", inp, tmp_path)
    co, ri, ewf = ref["column_offset"], ref["row_indices"], ref["edge_weight_forward"]
    ro, ci, ewb = ref["row_offset"], ref["column_indices"], ref["edge_weight_backward"]

    # PartitionToChunks + nts_norm_degree: CSC identical; CSR identical up to the order of the
    # destinations inside a source row, which the reference's loader leaves to thread arrival order.
    ch = oracle_chunk(inp)
    assert np.array_equal(ch["co"], co) and np.array_equal(ch["ri"], ri)
    assert ch["ewf"].tobytes() == ewf.tobytes()
    assert np.array_equal(ch["ro"], ro)
    a, b = rows_as_sorted_pairs(ro, ch["ci"], ch["ewb"]), rows_as_sorted_pairs(ro, ci, ewb)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])

    # ForwardCPUfuseOp: the oracle's fused (FMA) aggregation on the same arrays, bit for bit.
    x = inp["x"]
    assert oracle.spmm(x, ewf, co, ri, V, fused=True).tobytes() == ref["cpu_fwd"].tobytes()
    assert oracle.spmm(x, ewb, ro, ci, V, fused=True).tobytes() == ref["cpu_bwd"].tobytes()

    # SingleCPUSrcDstScatterOp: forward is a copy; backward adds with atomic compare-and-swap from
    # parallel threads, so its summation order is not defined -> tolerance.
    assert oracle.scatter_src_dst(x, x, co, ri).tobytes() == ref["cpu_scatter"].tobytes()
    want = sum(oracle.scatter_src_dst_bwd(inp["g2"], co, ri, V))  # source part + destination part
    scale = sum(oracle.scatter_src_dst_bwd(np.abs(inp["g2"]), co, ri, V))
    check(ref["cpu_scatter_bwd"], want, scale)

    # SingleCPUDstAggregateOp: one thread per destination adds its edges in order -> exact.
    assert oracle.aggregate_dst(inp["e"], co).tobytes() == ref["cpu_agg"].tobytes()
    assert oracle.scatter_dst(x, co, E).tobytes() == ref["cpu_agg_bwd"].tobytes()

    # SingleEdgeSoftMax calls libtorch's softmax per destination slice; the oracle restates the
    # stable textbook form, so the two agree to rounding, not bit for bit.
    y = oracle.edge_softmax(inp["m"], co)
    assert np.max(np.abs(y - ref["cpu_softmax"])) <= 4e-7
    assert np.max(np.abs(y - ref["cpu_softmax"]) / np.maximum(ref["cpu_softmax"], 1e-30)) <= 1e-5
    m1, gm1 = np.ascontiguousarray(inp["m"][:, :1]), np.ascontiguousarray(inp["gm"][:, :1])
    y1 = oracle.edge_softmax(m1, co)
    assert np.max(np.abs(y1 - ref["cpu_softmax1"])) <= 4e-7
    gx = oracle.edge_softmax_bwd(gm1, ref["cpu_softmax1"], co)
    assert np.max(np.abs(gx - ref["cpu_softmax1_bwd"])) <= 2e-6


@pytest.mark.gpu
@pytest.mark.skipif(not refops.available("gpu"), reason="reference-built GPU operator program not present")
@pytest.mark.parametrize("V,E,F,H,seed", CASES + [(40000, 900000, 128, 4, 4)])
def test_reference_gpu_operator_classes_over_the_library_match_its_cpu_operators(tmp_path, V, E, F, H, seed):
    """The reference's ForwardSingleGPUfuseOp, DistGPUScatterSrc/Dst, DistGPUEdgeSoftMax and
    DistGPUAggregateDst, unchanged, call Cuda_Stream of the HIP veneer -> libntship; their results
    are compared with the reference's CPU operators run in the same process on the same graph."""
    inp = refops.make_inputs(V, E, F, H, seed)
    ref = refops.run("gpu", "both", inp, tmp_path)
    co, ri = ref["column_offset"], ref["row_indices"]
    # aggregation: one wave walks a row's edges in order with fused multiply-adds, as nts_comp does ->
    # bit-identical; rows longer than the piece length are summed in pieces (calls of >= 65,536 edges) ->
    # tolerance for those
    x = inp["x"]
    for got, want, off, idx, w in ((ref["gpu_fwd"], ref["cpu_fwd"], co, ri, ref["edge_weight_forward"]),
                                   (ref["gpu_bwd"], ref["cpu_bwd"], ref["row_offset"], ref["column_indices"],
                                    ref["edge_weight_backward"])):
        one_wave = np.diff(off.astype(np.int64)) <= (planless_piece_edges(E) or E)
        assert got[one_wave].tobytes() == want[one_wave].tobytes()
        check(got, want, abs_term_scale(x, w, off, idx, V))
    # vertex -> edge copies
    assert ref["gpu_scatter_src"].tobytes() == ref["cpu_scatter"][:, :F].tobytes()
    assert ref["gpu_scatter_dst"].tobytes() == ref["cpu_scatter"][:, F:].tobytes()
    # their backward: mirror rows back to vertices, plus the destination part; the CPU operator's
    # own summation order is undefined (atomic adds from parallel threads) -> tolerance
    mi = ref["mirror_index"]
    has_out = np.diff(mi.astype(np.int64)) > 0
    got = ref["gpu_scatter_dst_bwd"].astype(np.float64)
    got[has_out] += ref["gpu_scatter_src_bwd"][mi[:-1][has_out]]
    scale = sum(oracle.scatter_src_dst_bwd(np.abs(inp["g2"]), co, ri, V))
    check(got.astype(np.float32), ref["cpu_scatter_bwd"], scale)
    # edge -> vertex sums in edge order, and the copy back
    # (rows of more than 1024 edges are summed by a whole block in slices -> tolerance for those)
    deg = np.diff(co.astype(np.int64))
    short = deg <= 1024
    assert ref["gpu_agg"][short].tobytes() == ref["cpu_agg"][short].tobytes()
    check(ref["gpu_agg"], ref["cpu_agg"], oracle.aggregate_dst(np.abs(inp["e"]), co))
    assert ref["gpu_agg_bwd"].tobytes() == ref["cpu_agg_bwd"].tobytes()
    # edge softmax against libtorch's softmax per slice: relative 1e-4 (fp32), as for every softmax test
    for name in ("softmax", "softmax1"):
        g, c = ref["gpu_" + name], ref["cpu_" + name]
        assert np.max(np.abs(g - c) / np.maximum(np.abs(c), 1e-30)) <= 1e-4, name
    # Softmax backward: gx = y*g - y*sum(g*y), each side using the y its own forward cached.  On hub
    # segments (10^4..10^5 edges) the two forward results differ by up to ~2e-5 relative (fp32
    # normaliser sums in different orders, inside the forward tolerance), and where y*g and y*sum(g*y)
    # cancel that common factor shows up amplified in gx.  So the GPU result is held to the exact
    # (fp64) value of the formula at its own y everywhere, and to the reference's CPU result on
    # segments of at most 1024 edges.
    seg = np.repeat(np.arange(V), deg)
    gm1 = np.ascontiguousarray(inp["gm"][:, :1])

    def exact(y):
        y64, g64 = y.astype(np.float64), gm1.astype(np.float64)
        dot = np.zeros(V)
        np.add.at(dot, seg, (y64 * g64)[:, 0])
        return y64 * g64 - y64 * dot[seg, None]

    y_gpu, y_cpu = ref["gpu_softmax1"], ref["cpu_softmax1"]
    scale = y_cpu * (np.abs(gm1) + oracle.aggregate_dst(np.abs(gm1) * y_cpu, co)[seg])
    check(ref["gpu_softmax1_bwd"], exact(y_gpu).astype(np.float32), scale)
    small = (deg <= 1024)[seg]
    check(ref["gpu_softmax1_bwd"][small], ref["cpu_softmax1_bwd"][small], scale[small])


@pytest.mark.skipif(not refops.available("gpu"), reason="reference-built program with sampCSC not present")
@pytest.mark.parametrize("V,E,batch,fanouts,seed", [(500, 6000, 40, [3, 5], 1), (20000, 300000, 512, [10, 25], 2),
                                                    (3000, 90000, 200, [5, 10, 15], 3)])
def test_oracle_matches_the_reference_sampled_layer_construction(tmp_path, V, E, batch, fanouts, seed):
    """sampCSC::postprocessing, generate_csr_from_csc, update_degree and compute_weight_forward /
    backward of the reference itself (core/coocsc.hpp:136-450), run on sampled lists made here, against
    the oracle's restatements: every array bit for bit."""
    _sampled_layers_case(tmp_path, V, E, batch, fanouts, seed, device_F=0)


@pytest.mark.gpu
@pytest.mark.skipif(not refops.available("gpu"), reason="reference-built program with sampCSC not present")
@pytest.mark.parametrize("V,E,batch,fanouts,seed", [(20000, 300000, 512, [10, 25], 2), (3000, 90000, 200, [15, 10, 5], 3)])
def test_reference_sampled_layers_on_the_device_match_the_oracle(tmp_path, V, E, batch, fanouts, seed):
    """The reference's sampCSC mirrors each layer on the device itself (grow-only arrays re-used from
    layer to layer, asynchronous copies: core/coocsc.hpp:673-773) through the veneer's allocator and
    copies, and the layer is aggregated forward and backward with the calls of SingleGPUSampleGraphOp
    (core/ntsMiniBatchGraphOp.hpp:288-375).  Results against the oracle's fused aggregation on the
    reference's own arrays: rows of at most one piece bit for bit, the rest within tolerance."""
    _sampled_layers_case(tmp_path, V, E, batch, fanouts, seed, device_F=24)


def _sampled_layers_case(tmp_path, V, E, batch, fanouts, seed, device_F):
    rng = np.random.default_rng(seed)
    gsrc = rng.integers(0, V, E).astype(np.uint32)
    gdst = np.minimum((rng.random(E) ** 2 * V).astype(np.uint32), V - 1)
    order = np.argsort(gdst, kind="stable")
    csc_src = gsrc[order]
    gco = np.concatenate([[0], np.cumsum(np.bincount(gdst, minlength=V))]).astype(np.int64)
    layers = []
    dst = rng.choice(V, batch, replace=False).astype(np.uint32)
    for fan in fanouts:
        co, picks = [0], []
        for d in dst:
            nb = csc_src[gco[d]:gco[d + 1]]
            take = nb if nb.size <= fan else nb[np.sort(rng.choice(nb.size, fan, replace=False))]
            picks.append(take)
            co.append(co[-1] + take.size)
        ri = np.concatenate(picks).astype(np.uint32) if picks else np.zeros(0, np.uint32)
        layers.append(dict(dst=dst, co=np.array(co, dtype=np.uint32), ri=ri))
        dst = np.unique(ri)  # the next hop's destinations are this hop's sources (ascending ids)
        if device_F:
            layers[-1]["x"] = rng.standard_normal((dst.size, device_F)).astype(np.float32)
            layers[-1]["g"] = rng.standard_normal((layers[-1]["dst"].size, device_F)).astype(np.float32)
    ref = refops.run_sampled_layers(gsrc, gdst, V, layers, tmp_path, device_F=device_F)
    for layer, want in zip(layers, ref):
        local, source, n_src = oracle.postprocess(layer["ri"], V)
        assert n_src == want["source"].size
        assert np.array_equal(source, want["source"]) and np.array_equal(local, want["row_indices"])
        ro, ci = oracle.csr_from_csc(layer["co"], local, n_src)
        assert np.array_equal(ro, want["row_offset"]) and np.array_equal(ci, want["column_indices"])
        outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
        ewf, ewb = oracle.layer_weights(layer["co"], local, ro, ci, source, layer["dst"], outd, ind)
        assert ewf.tobytes() == want["edge_weight_forward"].tobytes()
        assert ewb.tobytes() == want["edge_weight_backward"].tobytes()
        if device_F:
            Vd = layer["dst"].size
            for got, x, w, off, idx, rows in ((want["fwd"], layer["x"], ewf, layer["co"], local, Vd),
                                              (want["bwd"], layer["g"], ewb, ro, ci, n_src)):
                expect = oracle.spmm(x, w, off, idx, rows, fused=True)
                one_wave = np.diff(off.astype(np.int64)) <= (planless_piece_edges(idx.size) or idx.size)
                assert got[one_wave].tobytes() == expect[one_wave].tobytes()
                check(got, expect, abs_term_scale(x, w, off, idx, rows))
