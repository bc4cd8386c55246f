"""Runs the reference-built operator programs oracle/_ref/ref_fullgraph_{cpu,gpu} (the reference's
own loader, partitioner and operator classes behind oracle/ref_fullgraph_driver.cpp, built by
oracle/build_ref.sh where the reference tree is present) on seeded inputs and returns every array
they write.  Test infrastructure only."""
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = {k: os.path.join(ROOT, "oracle", "_ref", f"ref_fullgraph_{k}") for k in ("cpu", "gpu")}


def available(kind):
    return os.path.exists(PROGRAMS[kind])


def make_inputs(V, E, F, H, seed, skew=2.0):
    rng = np.random.default_rng(seed)
    src = np.minimum((rng.random(E) ** skew * V).astype(np.uint32), V - 1)
    dst = np.minimum((rng.random(E) ** (skew + 1) * V).astype(np.uint32), V - 1)
    return dict(src=src, dst=dst, x=rng.standard_normal((V, F)).astype(np.float32),
                m=(3 * rng.standard_normal((E, H))).astype(np.float32),
                gm=rng.standard_normal((E, H)).astype(np.float32),
                e=rng.standard_normal((E, F)).astype(np.float32),
                g2=rng.standard_normal((E, 2 * F)).astype(np.float32))


def run(kind, mode, inputs, tmp_path, timeout=600):
    """kind: which program ("cpu" / "gpu"); mode: "cpu", "gpu" or "both"."""
    V, F = inputs["x"].shape
    E, H = inputs["m"].shape
    prefix = os.path.join(str(tmp_path), "ref")
    np.stack([inputs["src"], inputs["dst"]], 1).astype(np.uint32).tofile(prefix + ".edge")
    for k in ("x", "m", "gm", "e", "g2"):
        inputs[k].tofile(prefix + "." + k)
    r = subprocess.run([PROGRAMS[kind], prefix + ".edge", str(V), str(F), str(H), prefix, mode], capture_output=True,
                       text=True, timeout=timeout)
    assert r.returncode == 0, f"reference program failed ({r.returncode}):\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}"
    out = {"stdout": r.stdout}
    shapes = {"column_offset": (np.uint32, (V + 1,)), "row_indices": (np.uint32, (E,)),
              "edge_weight_forward": (np.float32, (E,)), "row_offset": (np.uint32, (V + 1,)),
              "column_indices": (np.uint32, (E,)), "edge_weight_backward": (np.float32, (E,)),
              "mirror_index": (np.uint32, (V + 1,))}
    for side in ("cpu", "gpu"):
        shapes.update({f"{side}_fwd": (np.float32, (V, F)), f"{side}_bwd": (np.float32, (V, F)),
                       f"{side}_softmax": (np.float32, (E, H)), f"{side}_softmax1": (np.float32, (E, 1)),
                       f"{side}_softmax1_bwd": (np.float32, (E, 1)), f"{side}_agg": (np.float32, (V, F)),
                       f"{side}_agg_bwd": (np.float32, (E, F))})
    shapes.update({"cpu_scatter": (np.float32, (E, 2 * F)), "cpu_scatter_bwd": (np.float32, (V, F)),
                   "gpu_scatter_src": (np.float32, (E, F)), "gpu_scatter_dst": (np.float32, (E, F)),
                   "gpu_scatter_src_bwd": (np.float32, (-1, F)), "gpu_scatter_dst_bwd": (np.float32, (V, F))})
    for name, (dtype, shape) in shapes.items():
        path = prefix + "." + name
        if os.path.exists(path):
            out[name] = np.fromfile(path, dtype=dtype).reshape(shape)
    return out


def run_sampled_layers(graph_src, graph_dst, V, layers, tmp_path, timeout=600, device_F=0):
    """layers: list of dicts with dst [Vd], co [Vd+1], ri [E] (global source ids), uint32.  Runs the
    reference's sampCSC construction (the GPU-variant program; this mode makes no device call) and
    returns, per layer, source / row_indices / row_offset / column_indices / both weight arrays.
    With device_F > 0 (needs the GPU) every layer also carries x [src_size, F] and g [Vd, F]; the
    layers are then mirrored on the device by the reference's own sampCSC code and aggregated with
    the calls of SingleGPUSampleGraphOp, and "fwd" / "bwd" are returned as well."""
    prefix = os.path.join(str(tmp_path), "samp")
    np.stack([graph_src, graph_dst], 1).astype(np.uint32).tofile(prefix + ".edge")
    for k, layer in enumerate(layers):
        for name in ("dst", "co", "ri"):
            np.ascontiguousarray(layer[name], dtype=np.uint32).tofile(f"{prefix}.l{k}.{name}")
        if device_F:
            for name in ("x", "g"):
                np.ascontiguousarray(layer[name], dtype=np.float32).tofile(f"{prefix}.l{k}.{name}")
    r = subprocess.run([PROGRAMS["gpu"], prefix + ".edge", str(V), str(device_F or 4), str(len(layers)), prefix,
                        "mini" if device_F else "samp"], capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, f"reference program failed ({r.returncode}):\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}"
    out = []
    for k in range(len(layers)):
        d = {}
        for name, dtype in (("source", np.uint32), ("row_indices", np.uint32), ("row_offset", np.uint32),
                            ("column_indices", np.uint32), ("edge_weight_forward", np.float32),
                            ("edge_weight_backward", np.float32)):
            d[name] = np.fromfile(f"{prefix}.l{k}.{name}", dtype=dtype)
        if device_F:
            d["fwd"] = np.fromfile(f"{prefix}.l{k}.fwd", dtype=np.float32).reshape(-1, device_F)
            d["bwd"] = np.fromfile(f"{prefix}.l{k}.bwd", dtype=np.float32).reshape(-1, device_F)
        out.append(d)
    return out


def run_data_loader(V, F, classes, files_prefix, timeout=300):
    """Runs the reference's GNNDatum::readFeature_Label_Mask (GPU-variant program: its feature table
    lives in pinned memory) on <files_prefix>.feat / .label / .mask; needs <files_prefix>.edge."""
    r = subprocess.run([PROGRAMS["gpu"], files_prefix + ".edge", str(V), str(F), str(classes), files_prefix, "data"],
                       capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, f"reference program failed ({r.returncode}):\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}"
    width = classes if classes > 1 else 1
    return dict(local_feature=np.fromfile(files_prefix + ".local_feature", dtype=np.float32).reshape(V, F),
                local_label=np.fromfile(files_prefix + ".local_label", dtype=np.int64).reshape(V * width),
                global_label=np.fromfile(files_prefix + ".global_label", dtype=np.int64).reshape(V * width),
                local_mask=np.fromfile(files_prefix + ".local_mask", dtype=np.int32),
                global_mask=np.fromfile(files_prefix + ".global_mask", dtype=np.int32))
