"""ctypes binding of the CPU oracle (oracle/nts_oracle.c).

TEST INFRASTRUCTURE ONLY.  The oracle restates NeutronBench's own CPU graph operators and is the
checker the HIP path is compared against.  Only tests/, the smoke check and the cpu_baseline leg
of bench.py may import this package; the product package never does.

All functions take and return numpy arrays (uint32 indices, float32 values, int64 labels).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnts_oracle.so")
_lib = None

_u32p = ctypes.POINTER(ctypes.c_uint32)
_f32p = ctypes.POINTER(ctypes.c_float)
_i64p = ctypes.POINTER(ctypes.c_int64)


def build():
    """Compile oracle/libnts_oracle.so with gcc."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.nts_oracle_norm_degree.restype = ctypes.c_float
        _lib.nts_oracle_norm_degree.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        _lib.nts_oracle_postprocess.restype = ctypes.c_uint32
        _lib.nts_oracle_load_feature_cached.restype = ctypes.c_uint32
        _lib.nts_oracle_max_threads.restype = ctypes.c_int
    return _lib


def _u32(a):
    a = np.ascontiguousarray(a, dtype=np.uint32)
    return a, a.ctypes.data_as(_u32p)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _i64(a):
    a = np.ascontiguousarray(a, dtype=np.int64)
    return a, a.ctypes.data_as(_i64p)


def max_threads():
    return int(lib().nts_oracle_max_threads())


def norm_degree(out_deg, in_deg):
    return np.float32(lib().nts_oracle_norm_degree(int(out_deg), int(in_deg)))


def comp(output, inp, weight, fused=False):
    """nts_comp: returns output + inp * weight (a copy)."""
    out, po = _f32(np.array(output, dtype=np.float32, copy=True))
    x, px = _f32(inp)
    lib().nts_oracle_comp(po, px, ctypes.c_float(float(weight)), ctypes.c_uint32(out.size), ctypes.c_int(int(fused)))
    return out


def spmm(x, w, offsets, indices, rows, index_base=0, fused=False, threads=0):
    """Aggregation as a row gather: forward with CSC arrays, backward (pull) with CSR arrays."""
    x, px = _f32(x)
    F = x.shape[1]
    off, poff = _u32(offsets)
    idx, pidx = _u32(indices)
    pw = None
    if w is not None:
        w, pw = _f32(w)
    out = np.empty((rows, F), dtype=np.float32)
    lib().nts_oracle_spmm(px, out.ctypes.data_as(_f32p), pw, poff, pidx, ctypes.c_uint32(index_base),
                          ctypes.c_uint32(rows), ctypes.c_uint32(F), ctypes.c_int(int(fused)), ctypes.c_int(threads))
    return out


def spmm_push(gout, ewf, co, ri, Vs):
    gout, pg = _f32(gout)
    F = gout.shape[1]
    Vd = gout.shape[0]
    ewf, pw = _f32(ewf)
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    gin = np.empty((Vs, F), dtype=np.float32)
    lib().nts_oracle_spmm_push(pg, gin.ctypes.data_as(_f32p), pw, pco, pri, ctypes.c_uint32(Vd), ctypes.c_uint32(Vs),
                               ctypes.c_uint32(F))
    return gin


def degrees(coo_src, coo_dst, V):
    s, ps = _u32(coo_src)
    d, pd = _u32(coo_dst)
    outd = np.empty(V, dtype=np.uint32)
    ind = np.empty(V, dtype=np.uint32)
    lib().nts_oracle_degrees(ps, pd, ctypes.c_uint64(s.size), ctypes.c_uint32(V), outd.ctypes.data_as(_u32p),
                             ind.ctypes.data_as(_u32p))
    return outd, ind


def build_chunk(coo_src, coo_dst, V, out_degree, in_degree):
    """Full-graph CSC + CSR + GCN weights of one partition (PartitionToChunks)."""
    s, ps = _u32(coo_src)
    d, pd = _u32(coo_dst)
    od, pod = _u32(out_degree)
    idg, pid = _u32(in_degree)
    E = s.size
    co = np.empty(V + 1, dtype=np.uint32)
    ro = np.empty(V + 1, dtype=np.uint32)
    ri = np.empty(E, dtype=np.uint32)
    ci = np.empty(E, dtype=np.uint32)
    ewf = np.empty(E, dtype=np.float32)
    ewb = np.empty(E, dtype=np.float32)
    lib().nts_oracle_build_chunk(ps, pd, ctypes.c_uint64(E), ctypes.c_uint32(V), pod, pid, co.ctypes.data_as(_u32p),
                                 ri.ctypes.data_as(_u32p), ewf.ctypes.data_as(_f32p), ro.ctypes.data_as(_u32p),
                                 ci.ctypes.data_as(_u32p), ewb.ctypes.data_as(_f32p))
    return dict(co=co, ri=ri, ewf=ewf, ro=ro, ci=ci, ewb=ewb)


def postprocess(row_indices_global, V):
    """Returns (local row_indices, source, src_size)."""
    ri = np.array(row_indices_global, dtype=np.uint32, copy=True)
    source = np.empty(max(ri.size, 1), dtype=np.uint32)
    node_idx = np.zeros(V, dtype=np.uint32)
    n = lib().nts_oracle_postprocess(ri.ctypes.data_as(_u32p), ctypes.c_uint32(ri.size), ctypes.c_uint32(V),
                                     source.ctypes.data_as(_u32p), node_idx.ctypes.data_as(_u32p))
    return ri, source[:n].copy(), int(n)


def csr_from_csc(co, ri, Vs):
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    Vd = co.size - 1
    E = ri.size
    ro = np.empty(Vs + 1, dtype=np.uint32)
    ci = np.empty(E, dtype=np.uint32)
    lib().nts_oracle_csr_from_csc(pco, pri, ctypes.c_uint32(Vd), ctypes.c_uint32(Vs), ctypes.c_uint32(E),
                                  ro.ctypes.data_as(_u32p), ci.ctypes.data_as(_u32p))
    return ro, ci


def layer_weights(co, ri, ro, ci, source, destination, out_degree, in_degree):
    """update_degree + compute_weight_forward/backward; out_degree / in_degree are modified in place."""
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    ro, pro = _u32(ro)
    ci, pci = _u32(ci)
    src, psrc = _u32(source)
    dst, pdst = _u32(destination)
    assert out_degree.dtype == np.uint32 and in_degree.dtype == np.uint32
    E = ri.size
    ewf = np.empty(E, dtype=np.float32)
    ewb = np.empty(E, dtype=np.float32)
    lib().nts_oracle_layer_weights(pco, pri, pro, pci, psrc, pdst, ctypes.c_uint32(co.size - 1),
                                   ctypes.c_uint32(ro.size - 1), out_degree.ctypes.data_as(_u32p),
                                   in_degree.ctypes.data_as(_u32p), ewf.ctypes.data_as(_f32p),
                                   ewb.ctypes.data_as(_f32p))
    return ewf, ewb


def init_co(graph_co, dst, fanout):
    g, pg = _u32(graph_co)
    d, pd = _u32(dst)
    co = np.empty(d.size + 1, dtype=np.uint32)
    lib().nts_oracle_init_co(pg, pd, ctypes.c_uint32(d.size), ctypes.c_int(int(fanout)), co.ctypes.data_as(_u32p))
    return co


def get_feature(whole, src):
    whole, pw = _f32(whole)
    src, ps = _u32(src)
    F = whole.shape[1]
    out = np.empty((src.size, F), dtype=np.float32)
    lib().nts_oracle_get_feature(out.ctypes.data_as(_f32p), pw, ps, ctypes.c_uint32(src.size), ctypes.c_uint32(F))
    return out


def get_label(whole, dst):
    whole, pw = _i64(whole)
    dst, pd = _u32(dst)
    classes = 1 if whole.ndim == 1 else whole.shape[1]
    shape = (dst.size,) if whole.ndim == 1 else (dst.size, classes)
    out = np.empty(shape, dtype=np.int64)
    lib().nts_oracle_get_label(out.ctypes.data_as(_i64p), pw, pd, ctypes.c_uint32(dst.size), ctypes.c_uint32(classes))
    return out


def mark_cache(V, order, n_cache):
    order, po = _u32(order)
    hashmap = np.empty(V, dtype=np.uint32)
    lib().nts_oracle_mark_cache(hashmap.ctypes.data_as(_u32p), ctypes.c_uint32(V), po, ctypes.c_uint32(n_cache))
    return hashmap


def fill_cache(feature, order, n_cache, hashmap):
    feature, pf = _f32(feature)
    order, po = _u32(order)
    hashmap, ph = _u32(hashmap)
    F = feature.shape[1]
    cache = np.zeros((n_cache, F), dtype=np.float32)
    lib().nts_oracle_fill_cache(cache.ctypes.data_as(_f32p), pf, po, ctypes.c_uint32(n_cache), ph, ctypes.c_uint32(F))
    return cache


def load_feature_cached(feature, cache, source, hashmap):
    """Returns (batch features, hit positions, miss positions)."""
    feature, pf = _f32(feature)
    cache, pc = _f32(cache)
    source, ps = _u32(source)
    hashmap, ph = _u32(hashmap)
    F = feature.shape[1]
    n = source.size
    out = np.empty((n, F), dtype=np.float32)
    miss = np.empty(max(n, 1), dtype=np.uint32)
    hit = np.empty(max(n, 1), dtype=np.uint32)
    nh = lib().nts_oracle_load_feature_cached(out.ctypes.data_as(_f32p), pf, pc, ps, ctypes.c_uint32(n), ph,
                                              ctypes.c_uint32(F), miss.ctypes.data_as(_u32p),
                                              hit.ctypes.data_as(_u32p))
    return out, hit[:nh].copy(), miss[: n - nh].copy()


def scatter_src_dst(x_src, x_dst, co, ri):
    x_src, pxs = _f32(x_src)
    x_dst, pxd = _f32(x_dst)
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    F = x_src.shape[1]
    msg = np.empty((ri.size, 2 * F), dtype=np.float32)
    lib().nts_oracle_scatter_src_dst(msg.ctypes.data_as(_f32p), pxs, pxd, pco, pri, ctypes.c_uint32(co.size - 1),
                                     ctypes.c_uint32(F))
    return msg


def scatter_src_dst_bwd(g_msg, co, ri, Vs):
    g_msg, pg = _f32(g_msg)
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    F = g_msg.shape[1] // 2
    Vd = co.size - 1
    g_src = np.empty((Vs, F), dtype=np.float32)
    g_dst = np.empty((Vd, F), dtype=np.float32)
    lib().nts_oracle_scatter_src_dst_bwd(g_src.ctypes.data_as(_f32p), g_dst.ctypes.data_as(_f32p), pg, pco, pri,
                                         ctypes.c_uint32(Vd), ctypes.c_uint32(Vs), ctypes.c_uint32(F))
    return g_src, g_dst


def scatter_src(x_src, co, ri, mirror=None):
    x_src, px = _f32(x_src)
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    pm = None
    if mirror is not None:
        mirror, pm = _u32(mirror)
    F = x_src.shape[1]
    msg = np.empty((ri.size, F), dtype=np.float32)
    lib().nts_oracle_scatter_src(msg.ctypes.data_as(_f32p), px, pco, pri, pm, ctypes.c_uint32(co.size - 1),
                                 ctypes.c_uint32(F))
    return msg


def gather_to_src(g_msg, co, ri, Vs):
    g_msg, pg = _f32(g_msg)
    co, pco = _u32(co)
    ri, pri = _u32(ri)
    F = g_msg.shape[1]
    out = np.empty((Vs, F), dtype=np.float32)
    lib().nts_oracle_gather_to_src(out.ctypes.data_as(_f32p), pg, pco, pri, ctypes.c_uint32(co.size - 1),
                                   ctypes.c_uint32(Vs), ctypes.c_uint32(F))
    return out


def scatter_dst(x_dst, co, E):
    x_dst, px = _f32(x_dst)
    co, pco = _u32(co)
    F = x_dst.shape[1]
    msg = np.empty((E, F), dtype=np.float32)
    lib().nts_oracle_scatter_dst(msg.ctypes.data_as(_f32p), px, pco, ctypes.c_uint32(co.size - 1), ctypes.c_uint32(F))
    return msg


def aggregate_dst(msg, co):
    msg, pm = _f32(msg)
    co, pco = _u32(co)
    F = msg.shape[1]
    Vd = co.size - 1
    out = np.empty((Vd, F), dtype=np.float32)
    lib().nts_oracle_aggregate_dst(out.ctypes.data_as(_f32p), pm, pco, ctypes.c_uint32(Vd), ctypes.c_uint32(F))
    return out


def edge_softmax(x, co):
    x, px = _f32(x)
    co, pco = _u32(co)
    H = x.shape[1]
    y = np.zeros_like(x)
    lib().nts_oracle_edge_softmax(y.ctypes.data_as(_f32p), px, pco, ctypes.c_uint32(co.size - 1), ctypes.c_uint32(H))
    return y


def edge_softmax_bwd(gy, y, co):
    gy, pg = _f32(gy)
    y, py = _f32(y)
    co, pco = _u32(co)
    H = y.shape[1]
    gx = np.zeros_like(y)
    lib().nts_oracle_edge_softmax_bwd(gx.ctypes.data_as(_f32p), pg, py, pco, ctypes.c_uint32(co.size - 1),
                                      ctypes.c_uint32(H))
    return gx


def read_feature_label_mask(path_f, path_l, path_m, V, F, classes=1):
    """GNNDatum::readFeature_Label_Mask for one partition owning [0, V).  Returns a dict of the five tables."""
    width = classes if classes > 1 else 1
    feat = np.zeros((V, F), dtype=np.float32)
    ll = np.zeros(V * width, dtype=np.int64)
    gl = np.zeros(V * width, dtype=np.int64)
    lm = np.zeros(V, dtype=np.int32)
    gm = np.zeros(V, dtype=np.int32)
    i32p = ctypes.POINTER(ctypes.c_int32)
    rc = lib().nts_oracle_read_feature_label_mask(
        os.fsencode(path_f), os.fsencode(path_l), os.fsencode(path_m), ctypes.c_uint32(V), ctypes.c_uint32(F),
        ctypes.c_uint32(classes), feat.ctypes.data_as(_f32p), ll.ctypes.data_as(_i64p), lm.ctypes.data_as(i32p),
        gl.ctypes.data_as(_i64p), gm.ctypes.data_as(i32p))
    if rc != 0:
        raise IOError(f"oracle reader failed with {rc}")
    return dict(local_feature=feat, local_label=ll, local_mask=lm, global_label=gl, global_mask=gm)


def read_feature_label_mask_ogb(path_f, path_l, dir_m, V, F):
    feat = np.zeros((V, F), dtype=np.float32)
    ll = np.zeros(V, dtype=np.int64)
    lm = np.zeros(V, dtype=np.int32)
    rc = lib().nts_oracle_read_feature_label_mask_ogb(
        os.fsencode(path_f), os.fsencode(path_l), os.fsencode(dir_m), ctypes.c_uint32(V), ctypes.c_uint32(F),
        feat.ctypes.data_as(_f32p), ll.ctypes.data_as(_i64p), lm.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
    if rc != 0:
        raise IOError(f"oracle reader failed with {rc}")
    return dict(local_feature=feat, local_label=ll, local_mask=lm)


def read_edges(path):
    E = os.path.getsize(path) // 8
    src = np.empty(max(E, 1), dtype=np.uint32)
    dst = np.empty(max(E, 1), dtype=np.uint32)
    f = lib().nts_oracle_read_edges
    f.restype = ctypes.c_uint64
    n = f(os.fsencode(path), src.ctypes.data_as(_u32p), dst.ctypes.data_as(_u32p), ctypes.c_uint64(E))
    return src[:n].copy(), dst[:n].copy()
