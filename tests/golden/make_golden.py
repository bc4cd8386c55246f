#!/usr/bin/env python3
"""Writes tests/golden/exact_cases.json: small graphs whose expected results are exact.

The reference ships no golden vectors for this path, so these are constructed cases: every
out-degree * in-degree product is a perfect square and features are small integers, hence GCN
weights are exact reciprocals of integers that are powers of two, and every sum is exactly
representable in fp32 whatever the order of additions.  Expected values are computed here with
Python integers and Fractions only (no floating-point formulas, no project code), so the file pins
the layout conventions (edge order inside CSC / CSR rows, which end's degree enters the weight) and
the aggregation itself.

Run:  python tests/golden/make_golden.py
"""
import json
import math
import os
import random
from fractions import Fraction


def star_graph(hubs):
    """hubs: list of (hub id, leaf ids).  Every leaf has one edge to the hub and one edge from it."""
    edges = []
    for hub, leaves in hubs:
        for leaf in leaves:
            edges.append((leaf, hub))
            edges.append((hub, leaf))
    return edges


def layout(edges, V):
    coo = sorted(range(len(edges)), key=lambda j: edges[j][0])  # stable: by source, file order kept
    coo = [edges[j] for j in coo]
    out_deg = [max(1, sum(1 for s, _ in coo if s == v)) for v in range(V)]
    in_deg = [max(1, sum(1 for _, d in coo if d == v)) for v in range(V)]

    def weight(s, d):
        prod = out_deg[s] * in_deg[d]
        root = math.isqrt(prod)
        assert root * root == prod and (root & (root - 1)) == 0, "case must keep weights exact powers of two"
        return Fraction(1, root)

    co, ri, ewf = [0], [], []
    for v in range(V):
        for s, d in coo:
            if d == v:
                ri.append(s)
                ewf.append(weight(s, d))
        co.append(len(ri))
    ro, ci, ewb = [0], [], []
    for v in range(V):
        for s, d in coo:
            if s == v:
                ci.append(d)
                ewb.append(weight(s, d))
        ro.append(len(ci))
    return dict(co=co, ri=ri, ewf=ewf, ro=ro, ci=ci, ewb=ewb, out_deg=out_deg, in_deg=in_deg, coo=coo)


def spmm(x, w, off, idx, rows, F):
    out = []
    for r in range(rows):
        acc = [Fraction(0)] * F
        for e in range(off[r], off[r + 1]):
            acc = [a + w[e] * Fraction(v) for a, v in zip(acc, x[idx[e]])]
        out.append(acc)
    return out


def as_float(m):
    return [[float(v) for v in row] for row in m]


def main():
    rnd = random.Random(7)
    cases = []
    specs = [
        ("star4", 6, [(0, [1, 2, 3, 4])], 3),                     # hub degree 4, vertex 5 isolated
        ("star16_star4", 23, [(0, list(range(1, 17))), (17, [18, 19, 20, 21])], 5),  # vertex 22 isolated
        ("star64", 65, [(3, [v for v in range(65) if v != 3])], 2),
    ]
    for name, V, hubs, F in specs:
        edges = star_graph(hubs)
        rnd.shuffle(edges)
        lay = layout(edges, V)
        x = [[rnd.randint(-8, 8) for _ in range(F)] for _ in range(V)]
        y = spmm(x, lay["ewf"], lay["co"], lay["ri"], V, F)
        g = spmm(y, lay["ewb"], lay["ro"], lay["ci"], V, F)
        cases.append(dict(
            name=name, V=V, F=F,
            edges_src=[s for s, _ in edges], edges_dst=[d for _, d in edges],
            column_offset=lay["co"], row_indices=lay["ri"], edge_weight_forward=[float(w) for w in lay["ewf"]],
            row_offset=lay["ro"], column_indices=lay["ci"], edge_weight_backward=[float(w) for w in lay["ewb"]],
            out_degree=lay["out_deg"], in_degree=lay["in_deg"],
            x=x, forward=as_float(y), backward_of_forward=as_float(g)))
    # edge softmax: equal logits in segments of 1, 2, 4, 8 edges (and one empty segment) give 1/n exactly
    seg = [1, 2, 0, 4, 8]
    co = [0]
    for n in seg:
        co.append(co[-1] + n)
    H = 2
    logits, alpha = [], []
    for n in seg:
        base = [rnd.randint(-20, 20) for _ in range(H)]
        for _ in range(n):
            logits.append([float(b) for b in base])
            alpha.append([1.0 / n] * H)
    softmax = dict(column_offset=co, H=H, logits=logits, alpha=alpha)
    out = dict(comment="exact expected values; see make_golden.py", aggregation=cases, edge_softmax=softmax)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "exact_cases.json")
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
