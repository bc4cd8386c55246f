"""Oracle and HIP path against the committed exact-value fixtures (tests/golden/exact_cases.json,
written by tests/golden/make_golden.py with integer / Fraction arithmetic only)."""
import json
import os

import numpy as np
import pytest

import oracle

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "exact_cases.json")
GOLD = json.load(open(_PATH))


def _coo(case):
    src = np.array(case["edges_src"], dtype=np.int64)
    dst = np.array(case["edges_dst"], dtype=np.int64)
    order = np.argsort(src, kind="stable")
    return src[order].astype(np.uint32), dst[order].astype(np.uint32)


@pytest.mark.parametrize("case", GOLD["aggregation"], ids=lambda c: c["name"])
def test_oracle_matches_exact_fixture(case):
    V = case["V"]
    s, d = _coo(case)
    outd, ind = oracle.degrees(s, d, V)
    assert list(outd) == case["out_degree"] and list(ind) == case["in_degree"]
    ch = oracle.build_chunk(s, d, V, outd, ind)
    for key, name in (("co", "column_offset"), ("ri", "row_indices"), ("ro", "row_offset"), ("ci", "column_indices")):
        assert list(ch[key]) == case[name], name
    assert list(ch["ewf"]) == case["edge_weight_forward"] and list(ch["ewb"]) == case["edge_weight_backward"]
    x = np.array(case["x"], dtype=np.float32)
    for fused in (False, True):
        y = oracle.spmm(x, ch["ewf"], ch["co"], ch["ri"], V, fused=fused)
        assert np.array_equal(y, np.array(case["forward"], dtype=np.float32))
        g = oracle.spmm(y, ch["ewb"], ch["ro"], ch["ci"], V, fused=fused)
        assert np.array_equal(g, np.array(case["backward_of_forward"], dtype=np.float32))


def test_oracle_softmax_matches_exact_fixture():
    sm = GOLD["edge_softmax"]
    y = oracle.edge_softmax(np.array(sm["logits"], dtype=np.float32), np.array(sm["column_offset"], dtype=np.uint32))
    assert np.array_equal(y, np.array(sm["alpha"], dtype=np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLD["aggregation"], ids=lambda c: c["name"])
def test_hip_matches_exact_fixture(device, case):
    import torch

    from gpu_util import host_u32
    from neutronbench_amd.layout import FullGraphChunk
    from neutronbench_amd.ops import ForwardSingleGPUfuseOp

    V = case["V"]
    src = torch.tensor(case["edges_src"], dtype=torch.int64, device=device)
    dst = torch.tensor(case["edges_dst"], dtype=torch.int64, device=device)
    for chunk_edges in (0, 5):  # default schedule, and one that splits the hub rows
        chunk = FullGraphChunk.from_edges(src, dst, V, chunk_edges)
        assert list(host_u32(chunk.column_offset_gpu)) == case["column_offset"]
        assert list(host_u32(chunk.row_indices_gpu)) == case["row_indices"]
        assert list(host_u32(chunk.row_offset_gpu)) == case["row_offset"]
        assert list(host_u32(chunk.column_indices_gpu)) == case["column_indices"]
        assert chunk.edge_weight_forward_gpu.cpu().tolist() == case["edge_weight_forward"]
        assert chunk.edge_weight_backward_gpu.cpu().tolist() == case["edge_weight_backward"]
        op = ForwardSingleGPUfuseOp(chunk)
        x = torch.tensor(case["x"], dtype=torch.float32, device=device)
        y = op.forward(x)
        assert y.cpu().tolist() == case["forward"]
        assert op.backward(y).cpu().tolist() == case["backward_of_forward"]


@pytest.mark.gpu
def test_hip_softmax_matches_exact_fixture(device):
    import torch

    from neutronbench_amd.abi import call, ptr

    sm = GOLD["edge_softmax"]
    x = torch.tensor(sm["logits"], dtype=torch.float32, device=device)
    co = torch.tensor(sm["column_offset"], dtype=torch.int32, device=device)
    y = torch.full_like(x, float("nan"))
    call("nts_edge_softmax_fwd", ptr(y), ptr(x), ptr(co), co.numel() - 1, sm["H"], torch.cuda.current_stream().cuda_stream)
    assert y.cpu().tolist() == sm["alpha"]
