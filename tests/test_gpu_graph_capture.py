"""The aggregation and edge-softmax entry points launch kernels only (no allocation, no memset node,
no host synchronisation once the plan's scratch is reserved), so they can be recorded into a HIP
graph.  Every replay is checked against the eager result, with eager work in between."""
import numpy as np
import pytest
import torch

from gpu_util import dev
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.layout import SpmmPlan
from util import random_block

pytestmark = pytest.mark.gpu


def test_planned_aggregation_and_softmax_in_a_hip_graph(device):
    Vd, Vs, F, H = 600, 900, 100, 4
    co, ri = random_block(Vd, Vs, 15, seed=1, hub=2000, dup=True)
    for d in range(Vd):
        ri[co[d]:co[d + 1]] = np.sort(ri[co[d]:co[d + 1]])
    E = ri.size
    rng = np.random.default_rng(2)
    dco, dri = dev(co, device), dev(ri, device)
    w = dev(rng.random(E).astype(np.float32), device)
    x = torch.zeros(Vs, F, device=device)
    out = torch.zeros(Vd, F, device=device)
    logits = torch.zeros(E, H, device=device)
    alpha = torch.zeros(E, H, device=device)
    plan = SpmmPlan(dco, Vd, E, 64, dri, Vs, 4)
    plan.reserve(F)  # scratch allocated before the capture

    def run():
        s = torch.cuda.current_stream().cuda_stream
        call("nts_spmm_gather_planned", plan.handle, ptr(x), ptr(out), ptr(w), ptr(dco), ptr(dri), 0, F, 0, s)
        call("nts_edge_softmax_fwd", ptr(alpha), ptr(logits), ptr(dco), Vd, H, s)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run()
    for rep in range(4):
        x.copy_(torch.from_numpy(rng.standard_normal((Vs, F)).astype(np.float32)))
        logits.copy_(torch.from_numpy(rng.standard_normal((E, H)).astype(np.float32)))
        graph.replay()
        torch.cuda.synchronize()
        got_out, got_alpha = out.clone(), alpha.clone()
        out.zero_()
        alpha.zero_()
        run()  # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got_out, out), f"replay {rep}: aggregation differs from the eager launch"
        assert torch.equal(got_alpha, alpha), f"replay {rep}: softmax differs from the eager launch"
        assert float(out.abs().sum()) > 0
    # An eager call on another stream after the capture: the captured call left no event behind that
    # this one would wait on (a wait on an event recorded under capture is an error), and once the
    # caller has ordered the streams the result is the eager one again.
    torch.cuda.synchronize()
    other = torch.cuda.Stream()
    with torch.cuda.stream(other):
        call("nts_spmm_gather_planned", plan.handle, ptr(x), ptr(out), ptr(w), ptr(dco), ptr(dri), 0, F, 0,
             other.cuda_stream)
    other.synchronize()
    want = out.clone()
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    plan.close()
