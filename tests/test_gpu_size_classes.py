"""Segment-size classes of the per-destination kernels: every boundary between the short-group,
wave (register-resident / multi-pass), block and piece paths is hit exactly, for several head
counts and widths, and compared with the formulas evaluated in fp64 (the sequential fp32 oracle is
itself ~2e-4 off on 10^5-value segments)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, stream
from neutronbench_amd.abi import call, ptr
from util import check

pytestmark = pytest.mark.gpu


def boundary_graph(values_per_edge, rng, Vd=20000):
    """Degrees around every class boundary (in values = edges * values_per_edge), plus empty rows,
    tiny rows and Poisson filler; returns co (uint32) and the destination of every edge."""
    w = values_per_edge
    marks = []
    for limit in (128, 512, 32768, 131072):           # softmax classes, in values
        for n in (limit - w, limit, limit + w):
            marks.append(max(n // w, 0))
    for limit in (1024, 16384):                       # edge-sum classes, in edges
        marks += [limit - 1, limit, limit + 1]
    marks += [0, 0, 1, 2, 3, 64, 65, 40000]
    deg = rng.poisson(3, Vd).astype(np.int64)
    pos = rng.choice(Vd, len(marks), replace=False)
    deg[pos] = marks
    co = np.concatenate([[0], np.cumsum(deg)]).astype(np.uint32)
    seg = np.repeat(np.arange(Vd), deg)
    return co, seg, deg


def seg_sum(v, seg, Vd):
    out = np.zeros((Vd,) + v.shape[1:])
    np.add.at(out, seg, v)
    return out


@pytest.mark.parametrize("H", [1, 2, 4, 16, 64, 3])
def test_softmax_and_attention_across_size_classes(device, H):
    print(f"case H={H}", flush=True)
    rng = np.random.default_rng(1000 + H)
    co, seg, deg = boundary_graph(H, rng)
    Vd, E, Vs = deg.size, int(co[-1]), 5000
    x = (rng.standard_normal((E, H)) * 3).astype(np.float32)
    gy = rng.standard_normal((E, H)).astype(np.float32)
    ri = rng.integers(0, Vs, E).astype(np.uint32)
    dco, dri, dx, dgy = dev(co, device), dev(ri, device), dev(x, device), dev(gy, device)

    def softmax64(v):
        v = v.astype(np.float64)
        mx = np.full((Vd, H), -np.inf)
        np.maximum.at(mx, seg, v)
        ex = np.exp(v - mx[seg])
        return ex / seg_sum(ex, seg, Vd)[seg]

    y = torch.full((E, H), float("nan"), device=device)
    call("nts_edge_softmax_fwd", ptr(y), ptr(dx), ptr(dco), Vd, H, stream())
    got = y.cpu().numpy()
    assert not np.isnan(got).any()
    check(got, softmax64(x).astype(np.float32), scale=1.0, floor=1e-7)
    gx = torch.full((E, H), float("nan"), device=device)
    call("nts_edge_softmax_bwd", ptr(gx), ptr(dgy), ptr(y), ptr(dco), Vd, H, stream())
    y64, g64 = got.astype(np.float64), gy.astype(np.float64)
    want = y64 * (g64 - seg_sum(g64 * y64, seg, Vd)[seg])
    scale = y64 * (np.abs(g64) + seg_sum(np.abs(g64) * y64, seg, Vd)[seg])
    check(gx.cpu().numpy(), want.astype(np.float32), scale=scale.astype(np.float32))

    el = rng.standard_normal((Vs, H)).astype(np.float32)
    er = rng.standard_normal((Vd, H)).astype(np.float32)
    pre = el[ri] + er[seg]
    m = np.where(pre > 0, pre, np.float32(0.2) * pre).astype(np.float32)
    alpha_ref = softmax64(m)
    d_el, d_er = dev(el, device), dev(er, device)
    alpha = torch.full((E, H), float("nan"), device=device)
    call("nts_gat_attention_fwd", ptr(alpha), ptr(d_el), ptr(d_er), ptr(dco), ptr(dri), Vd, H, 0.2, stream())
    check(alpha.cpu().numpy(), alpha_ref.astype(np.float32), scale=1.0, floor=1e-7)
    d_alpha = dev(alpha_ref.astype(np.float32), device)
    a64 = alpha_ref.astype(np.float32).astype(np.float64)
    gs = torch.full((E, H), float("nan"), device=device)
    ger = torch.full((Vd, H), float("nan"), device=device)
    call("nts_gat_attention_bwd", ptr(gs), ptr(ger), ptr(dgy), ptr(d_alpha), ptr(d_el), ptr(d_er), ptr(dco), ptr(dri), Vd,
         H, 0.2, stream())
    gs_want = a64 * (g64 - seg_sum(g64 * a64, seg, Vd)[seg]) * np.where(pre > 0, 1.0, 0.2)
    gs_scale = a64 * (np.abs(g64) + seg_sum(np.abs(g64) * a64, seg, Vd)[seg])
    check(gs.cpu().numpy(), gs_want.astype(np.float32), scale=gs_scale.astype(np.float32))
    ger_got = ger.cpu().numpy()
    assert not np.isnan(ger_got).any()  # empty destinations get zeros
    check(ger_got, seg_sum(gs_want, seg, Vd).astype(np.float32), scale=seg_sum(gs_scale, seg, Vd).astype(np.float32))

    # The same call with every float array one float off a 16-byte boundary: the library may only use
    # 16-byte lanes when all of them allow it, and must give the same results when they do not.
    def off1(t):
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=t.device)
        view = buf[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == 4
        return view

    u_el, u_er, u_gy, u_alpha_in = off1(d_el), off1(d_er), off1(dgy), off1(d_alpha)
    u_alpha = off1(torch.full((E, H), float("nan"), device=device))
    call("nts_gat_attention_fwd", ptr(u_alpha), ptr(u_el), ptr(u_er), ptr(dco), ptr(dri), Vd, H, 0.2, stream())
    check(u_alpha.cpu().numpy(), alpha_ref.astype(np.float32), scale=1.0, floor=1e-7)
    u_gs = off1(torch.full((E, H), float("nan"), device=device))
    u_ger = off1(torch.full((Vd, H), float("nan"), device=device))
    call("nts_gat_attention_bwd", ptr(u_gs), ptr(u_ger), ptr(u_gy), ptr(u_alpha_in), ptr(u_el), ptr(u_er), ptr(dco),
         ptr(dri), Vd, H, 0.2, stream())
    check(u_gs.cpu().numpy(), gs_want.astype(np.float32), scale=gs_scale.astype(np.float32))
    check(u_ger.cpu().numpy(), seg_sum(gs_want, seg, Vd).astype(np.float32),
          scale=seg_sum(gs_scale, seg, Vd).astype(np.float32))


@pytest.mark.parametrize("F", [1, 2, 4, 8, 12, 16, 32, 100, 260])
def test_edge_sums_across_size_classes(device, F):
    print(f"case F={F}", flush=True)
    rng = np.random.default_rng(2000 + F)
    co, seg, deg = boundary_graph(1, rng)
    Vd, E = deg.size, int(co[-1])
    msg = rng.standard_normal((E, F)).astype(np.float32)
    dco, dmsg = dev(co, device), dev(msg, device)
    out = torch.full((Vd, F), float("nan"), device=device)
    call("nts_gather_edge_to_dst", ptr(out), ptr(dmsg), ptr(dco), Vd, F, 0, stream())
    got = out.cpu().numpy()
    assert not np.isnan(got).any()
    want = seg_sum(msg.astype(np.float64), seg, Vd)
    scale = seg_sum(np.abs(msg).astype(np.float64), seg, Vd)
    check(got, want.astype(np.float32), scale=scale.astype(np.float32))
    # rows of at most 1,024 edges are sequential chains: exactly the fp32 running sum
    # (also for rows of 16 to 64 bytes, whose loads are spread over eight lanes): every row above 8
    # edges, where a spread row takes more than one lane's loads, and 200 of the others
    chains = (deg > 0) & (deg <= 1024)
    for r in np.concatenate([np.flatnonzero(chains & (deg > 8)), np.flatnonzero(chains)[:200]]):
        acc = np.zeros(F, dtype=np.float32)
        for e in range(int(co[r]), int(co[r + 1])):
            acc = acc + msg[e]
        assert np.array_equal(got[r], acc), int(deg[r])
    init = rng.standard_normal((Vd, F)).astype(np.float32)
    out2 = dev(init, device)
    call("nts_gather_edge_to_dst", ptr(out2), ptr(dmsg), ptr(dco), Vd, F, 1, stream())
    check(out2.cpu().numpy(), (want + init).astype(np.float32), scale=(scale + np.abs(init)).astype(np.float32))
