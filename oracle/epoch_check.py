"""Checker for one mini-batch written out by the native epoch driver (lib/nts_epoch --dump-dir):
every array of the batch against the CPU oracle.  TEST INFRASTRUCTURE, like the rest of oracle/.

What is compared, and how:
  sampling      column_offset == init_co(graph, destination, fanout) (core/ntsSampler.hpp:843-921), every
                sampled source is an in-neighbour of its destination, a destination that keeps all its
                neighbours keeps them in CSC order                                    (exact)
  structure     local row_indices + source list == postprocess, CSR == csr_from_csc, both weight arrays
                == layer_weights (core/coocsc.hpp:136-216, 243-309, 338-424)            (bit for bit)
  gather        features == get_feature, labels == get_label, cache hits counted   (bit for bit)
  aggregation   forward and backward of every layer == spmm on the dumped input: rows of at most 256
                edges bit for bit against the fused chain, longer rows within
                1e-4 * max(|a|, |b|, 1e-2 * sum|terms|)
  GAT           alpha, attention-weighted aggregate, its two gradients, the fused attention backward and
                the per-source sums against the chain of the oracle's edge operators, same tolerance
"""
import json
import os

import numpy as np

import oracle

TOL = 1e-4


def _load(d, layer, name, dtype):
    return np.fromfile(os.path.join(d, f"L{layer}_{name}.bin"), dtype=dtype)


def _rel_err(got, ref, scale):
    den = np.maximum(np.maximum(np.abs(got), np.abs(ref)), 1e-2 * np.abs(scale) + 1e-30)
    return float((np.abs(got.astype(np.float64) - ref) / den).max()) if got.size else 0.0


def check_dump(dump_dir, graph_co, graph_ri, features, labels, fanouts, cache_fraction=0.0, slope=0.2):
    """graph_co / graph_ri: whole-graph CSC (uint32 numpy); features [V, F] float32; labels [V] int64;
    fanouts in hop order (the batch's own hop first).  Returns a dict with ok, the worst relative
    error, how many rows were equal bit for bit, and the first failure's name (or None)."""
    meta = json.load(open(os.path.join(dump_dir, "meta.json")))
    hops, H = meta["hops"], meta["heads"]
    V = graph_co.size - 1
    layers = []
    for l, m in enumerate(meta["layers"]):
        a = dict(m)
        for name in ("destination", "source", "column_offset", "row_indices", "row_offset", "column_indices"):
            a[name] = _load(dump_dir, l, name, np.uint32)
        for name in ("edge_weight_forward", "edge_weight_backward"):
            a[name] = _load(dump_dir, l, name, np.float32)
        if H:
            a["csr_to_csc"] = _load(dump_dir, l, "csr_to_csc", np.uint32)
        layers.append(a)
    res = {"ok": False, "failed": None, "max_rel_err": 0.0, "bit_exact_rows": 0, "checked_rows": 0,
           "sampled_edges": int(sum(a["e_size"] for a in layers)), "tolerance": TOL}

    def fail(what):
        res["failed"] = what
        return res

    # --- sampling and structure, hop by hop (the batch's own hop is the last layer) ---
    outd, ind = np.ones(V, np.uint32), np.ones(V, np.uint32)
    for hop in range(hops):
        l = hops - 1 - hop
        a = layers[l]
        co, ri, src, dst = a["column_offset"], a["row_indices"], a["source"], a["destination"]
        if co.size != a["v_size"] + 1 or ri.size != a["e_size"] or src.size != a["src_size"]:
            return fail(f"layer {l}: array sizes differ from the layer's shape")
        if not np.array_equal(co, oracle.init_co(graph_co, dst, fanouts[hop])):
            return fail(f"layer {l}: column_offset != init_co")
        glob = src[ri]
        deg = np.diff(co.astype(np.int64))
        owner = np.repeat(np.arange(dst.size), deg)
        lo, hi = graph_co[dst].astype(np.int64), graph_co[dst.astype(np.int64) + 1].astype(np.int64)
        # membership: the graph's CSC rows ascend, so a binary search inside the destination's row finds the source
        pos = lo[owner].copy()
        span = (hi - lo)[owner]
        step = 1 << max(int(span.max()).bit_length() - 1, 0) if span.size else 0
        while step:
            probe = pos + step
            ok = (probe < hi[owner]) & (graph_ri[np.minimum(probe, graph_ri.size - 1)] <= glob)
            pos = np.where(ok, probe, pos)
            step >>= 1
        if glob.size and not np.array_equal(graph_ri[pos], glob):
            return fail(f"layer {l}: a sampled source is not an in-neighbour of its destination")
        full = (hi - lo) == deg  # destinations that keep every neighbour: CSC order, all of them
        if full.any():
            sel = full[owner]
            want = np.concatenate([graph_ri[b:e] for b, e in zip(lo[full][:2000], hi[full][:2000])]) if full.any() else glob[:0]
            if not np.array_equal(glob[sel][:want.size], want):
                return fail(f"layer {l}: a fully kept neighbourhood is not in CSC order")
        local, source_ref, n = oracle.postprocess(glob, V)
        if n != src.size or not np.array_equal(source_ref, src) or not np.array_equal(local, ri):
            return fail(f"layer {l}: relabelled sources != postprocess")
        ro, ci = oracle.csr_from_csc(co, local, n)
        if not np.array_equal(ro, a["row_offset"]) or not np.array_equal(ci, a["column_indices"]):
            return fail(f"layer {l}: CSR != csr_from_csc")
        ewf, ewb = oracle.layer_weights(co, local, ro, ci, src, dst, outd, ind)
        if ewf.tobytes() != a["edge_weight_forward"].tobytes() or ewb.tobytes() != a["edge_weight_backward"].tobytes():
            return fail(f"layer {l}: edge weights != layer_weights")
        if hop + 1 < hops and not np.array_equal(layers[l - 1]["destination"], src):
            return fail(f"layer {l}: the next hop's destinations are not this hop's sources")

    # --- gather ---
    F = meta["F"]
    x = np.fromfile(os.path.join(dump_dir, "x.bin"), dtype=np.float32).reshape(-1, F)
    if x.tobytes() != oracle.get_feature(features, layers[0]["source"]).tobytes():
        return fail("gathered features != get_feature")
    lab = np.fromfile(os.path.join(dump_dir, "labels.bin"), dtype=np.int64)
    if not np.array_equal(lab, oracle.get_label(labels, layers[-1]["destination"])):
        return fail("gathered labels != get_label")
    if cache_fraction > 0:
        n_cache = int(cache_fraction * V)
        out_deg = np.bincount(graph_ri, minlength=V)
        order = np.argsort(-out_deg.astype(np.int64), kind="stable")[:n_cache].astype(np.uint32)
        hashmap = oracle.mark_cache(V, order, n_cache)
        hits = int((hashmap[layers[0]["source"]] != 0xFFFFFFFF).sum())
        if meta["cache_rows"] != n_cache or meta["cache_hits"] != hits:
            return fail(f"cache hits {meta['cache_hits']} != {hits}")
        res["cache_hits"] = hits
    res["gathered_rows"] = int(x.shape[0])

    def compare(name, got, ref, scale, exact_rows=None, fused=None):
        e = _rel_err(got, ref, scale)
        res["max_rel_err"] = max(res["max_rel_err"], e)
        res["checked_rows"] += int(got.shape[0])
        if e > TOL:
            res["failed"] = f"{name}: max rel err {e:.3e}"
            return False
        if exact_rows is not None and fused is not None:
            if got[exact_rows].tobytes() != fused[exact_rows].tobytes():
                res["failed"] = f"{name}: rows that are never cut differ from the fused chain"
                return False
            res["bit_exact_rows"] += int(exact_rows.sum())
        return True

    if not H:
        for l, a in enumerate(layers):
            w = a["width"]
            co, ri, ro, ci = a["column_offset"], a["row_indices"], a["row_offset"], a["column_indices"]
            ewf, ewb = a["edge_weight_forward"], a["edge_weight_backward"]
            xin = _load(dump_dir, l, "in", np.float32).reshape(a["src_size"], w)
            out = _load(dump_dir, l, "out", np.float32).reshape(a["v_size"], w)
            if l == 0 and xin.tobytes() != x.tobytes():
                return fail("layer 0 did not aggregate the gathered features")
            ref = oracle.spmm(xin, ewf, co, ri, a["v_size"])
            if not compare(f"layer {l} forward", out, ref, oracle.spmm(np.abs(xin), ewf, co, ri, a["v_size"]),
                           np.diff(co.astype(np.int64)) <= 256, oracle.spmm(xin, ewf, co, ri, a["v_size"], fused=True)):
                return res
            gout = _load(dump_dir, l, "gout", np.float32).reshape(a["v_size"], w)
            gin = _load(dump_dir, l, "gin", np.float32).reshape(a["src_size"], w)
            ref = oracle.spmm(gout, ewb, ro, ci, a["src_size"])
            if not compare(f"layer {l} backward", gin, ref, oracle.spmm(np.abs(gout), ewb, ro, ci, a["src_size"]),
                           np.diff(ro.astype(np.int64)) <= 256,
                           oracle.spmm(gout, ewb, ro, ci, a["src_size"], fused=True)):
                return res
        res["ok"] = True
        return res

    # --- GAT layers: the chain of the oracle's edge operators (toolkits/GAT_CPU.hpp:178-204) ---
    Fh = meta["hidden"] // H
    for l, a in enumerate(layers):
        Vd, Vs, E = a["v_size"], a["src_size"], a["e_size"]
        co, ri, ro, perm = a["column_offset"], a["row_indices"], a["row_offset"], a["csr_to_csc"]
        deg = np.diff(co.astype(np.int64))
        dst_of = np.repeat(np.arange(Vd), deg)
        xs = _load(dump_dir, l, "x", np.float32).reshape(Vs, H * Fh)
        el = _load(dump_dir, l, "el", np.float32).reshape(Vs, H)
        er = _load(dump_dir, l, "er", np.float32).reshape(Vd, H)
        alpha = _load(dump_dir, l, "alpha", np.float32).reshape(E, H)
        out = _load(dump_dir, l, "out", np.float32).reshape(Vd, H * Fh)
        pre = oracle.scatter_src(el, co, ri) + oracle.scatter_dst(er, co, E)
        score = np.where(pre > 0, pre, np.float32(slope) * pre).astype(np.float32)
        a_ref = oracle.edge_softmax(score, co)
        if not compare(f"layer {l} attention", alpha, a_ref, np.ones_like(a_ref)):
            return res
        msg = oracle.scatter_src(xs, co, ri)
        wmsg = (msg.reshape(E, H, Fh) * alpha[:, :, None]).reshape(E, H * Fh).astype(np.float32)
        if not compare(f"layer {l} weighted aggregate", out, oracle.aggregate_dst(wmsg, co),
                       oracle.aggregate_dst(np.abs(wmsg), co)):
            return res
        gout = _load(dump_dir, l, "gout", np.float32).reshape(Vd, H * Fh)
        gmsg = oracle.scatter_dst(gout, co, E)
        gin = _load(dump_dir, l, "gin", np.float32).reshape(Vs, H * Fh)
        gw = (gmsg.reshape(E, H, Fh) * alpha[:, :, None]).reshape(E, H * Fh).astype(np.float32)
        if not compare(f"layer {l} gradient of the features", gin, oracle.gather_to_src(gw, co, ri, Vs),
                       oracle.gather_to_src(np.abs(gw), co, ri, Vs)):
            return res
        galpha = _load(dump_dir, l, "galpha", np.float32).reshape(E, H)
        prod = msg.reshape(E, H, Fh).astype(np.float64) * gmsg.reshape(E, H, Fh)
        if not compare(f"layer {l} gradient of alpha", galpha, prod.sum(2), np.abs(prod).sum(2)):
            return res
        gs = _load(dump_dir, l, "gs", np.float32).reshape(E, H)
        slope_of = np.where(pre > 0, np.float32(1), np.float32(slope))
        gs_ref = oracle.edge_softmax_bwd(galpha, alpha, co) * slope_of
        seg = np.zeros((Vd, H))
        np.add.at(seg, dst_of, np.abs(alpha.astype(np.float64) * galpha))
        term = alpha * (np.abs(galpha) + seg[dst_of])
        if not compare(f"layer {l} gradient of the scores", gs, gs_ref, term):
            return res
        ger = _load(dump_dir, l, "ger", np.float32).reshape(Vd, H)
        gel = _load(dump_dir, l, "gel", np.float32).reshape(Vs, H)
        if not compare(f"layer {l} gradient of er", ger, oracle.aggregate_dst(gs, co),
                       oracle.aggregate_dst(term.astype(np.float32), co)):
            return res
        if not compare(f"layer {l} gradient of el", gel, oracle.gather_to_src(gs, co, ri, Vs),
                       oracle.gather_to_src(term.astype(np.float32), co, ri, Vs)):
            return res
        if not np.array_equal(np.sort(perm), np.arange(E, dtype=np.uint32)):
            return fail(f"layer {l}: csr_to_csc is not a permutation")
    res["ok"] = True
    return res
