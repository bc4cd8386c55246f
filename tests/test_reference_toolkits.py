"""The reference's own toolkit program, unchanged, over this library.

oracle/build_toolkits.sh compiles toolkits/main.cpp, core/GraphSegment.cpp and comm/network.cpp from the
reference tree with CUDA_ENABLE against neutronbench_amd/host/compat (the veneer in place of cuda/) and
links libntship.so and libtorch's ROCm build: oracle/_ref/nts.  The tests write an Arxiv-shaped
synthetic dataset with the library's own .edge / .feat / .label / .mask writers, a .cfg file, and run

  * GCNNEIGHBORGPU  (toolkits/GCN_GPU_NEIGHBOR.hpp: the reference's sampler, sampCSC device mirror,
                    zero-copy feature / label gather, SingleGPUSampleGraphOp, libtorch dense layers)
  * GCNEAGERSINGLE  (ForwardSingleGPUfuseOp on the full graph), GINGPU (ForwardGPUfuseOp: rows travel as
                    message records), GATGPUDIST (DistGPU* edge operators and edge softmax)

on the GPU (two epochs of the sampled toolkit, eight full-batch steps of the others); and oracle/_ref/ref_minibatch, which samples batches with the
reference's sampler and compares the reference's SingleGPUSampleGraphOp (over this library) with its
MiniBatchFuseOp (CPU) on every sampled layer, forward and backward, to 1e-4.

The programs are integration demonstrations: they are built with a METIS shim header (the reference's
submodule is empty) and pin nothing about the oracle.
"""
import math
import os
import re
import subprocess

import numpy as np
import pytest
import torch

from neutronbench_amd import dataset, synth

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NTS = os.path.join(ROOT, "oracle", "_ref", "nts")
MINI = os.path.join(ROOT, "oracle", "_ref", "ref_minibatch")
V, E, F, CLASSES = 169_343, 2_480_000, 128, 40


@pytest.fixture(scope="module")
def arxiv_shaped_files(device, tmp_path_factory):
    if not os.path.exists(NTS):
        pytest.skip("oracle/_ref/nts has not been built (oracle/build_toolkits.sh needs the reference tree)")
    d = str(tmp_path_factory.mktemp("arxiv_shaped"))
    src, dst = synth.rmat_edges(V, E, seed=2, device=device, sort=True)
    dataset.write_edge_file(os.path.join(d, "g.edge"), torch.stack([src, dst], 1).cpu().numpy())
    feat = synth.normal_features(V, F, seed=23)
    dataset.write_feature_file(os.path.join(d, "g.feat"), feat.numpy())
    # labels a model can learn: the largest of a vertex's first CLASSES features
    dataset.write_label_file(os.path.join(d, "g.label"), feat[:, :CLASSES].argmax(1).numpy())
    r = synth.uniform24(torch.arange(V), 77).numpy() / float(1 << 24)
    dataset.write_mask_file(os.path.join(d, "g.mask"), np.where(r < 0.537, 0, np.where(r < 0.713, 1, 2)))
    return d


def write_cfg(d, algorithm, **extra):
    lines = dict(ALGORITHM=algorithm, VERTICES=V, EPOCHS=2, LAYERS=f"{F}-128-{CLASSES}", FANOUT="10,25",
                 VALFANOUT="10,25", BATCH_SIZE=1024, BATCH_TYPE="shuffle", EDGE_FILE=f"{d}/g.edge",
                 FEATURE_FILE=f"{d}/g.feat", LABEL_FILE=f"{d}/g.label", MASK_FILE=f"{d}/g.mask", MINI_PULL=1,
                 CACHE_TYPE="none", PIPELINES=1, MODE="pipeline", CLASSES=1, PROC_OVERLAP=0, PROC_LOCAL=0, PROC_CUDA=0,
                 PROC_REP=0, LOCK_FREE=1, TIME_SKIP=0, RUNS=1, LEARN_RATE=0.01, WEIGHT_DECAY=0.0001, DECAY_RATE=0.97,
                 DECAY_EPOCH=100, DROP_RATE=0.5)
    lines.update(extra)
    path = os.path.join(d, f"{algorithm}{'_' + '_'.join(map(str, extra.values())) if extra else ''}.cfg")
    with open(path, "w") as f:
        f.write("".join(f"{k}:{v}\n" for k, v in lines.items()))
    return path


def run(program, *args, cwd):
    print(f"running {os.path.basename(program)} {' '.join(args)}", flush=True)
    p = subprocess.run([program, *args], capture_output=True, text=True, timeout=400, cwd=cwd)
    assert p.returncode == 0, f"exit {p.returncode}\n{p.stdout[-3000:]}\n{p.stderr[-2000:]}"
    return p.stdout


def test_reference_gpu_operator_equals_its_cpu_operator_on_sampled_layers(arxiv_shaped_files):
    d = arxiv_shaped_files
    out = run(MINI, write_cfg(d, "GCNNEIGHBORGPU"), "3", cwd=d)
    rows = re.findall(r"reference operators: batch (\d+) layer (\d+) v_size (\d+) e_size (\d+) src_size (\d+) F (\d+) "
                      r"forward_max_rel_err (\S+) forward_equal_rows (\d+) backward_max_rel_err (\S+) "
                      r"backward_equal_rows (\d+)", out)
    assert len(rows) == 6  # 3 batches x 2 layers
    for b, l, v, e, s, f, ef, sf, eb, sb in rows:
        print(f"batch {b} layer {l}: Vd={v} E={e} Vs={s} fwd {ef} ({sf} rows equal) bwd {eb} ({sb} rows equal)")
        assert float(ef) <= 1e-4 and float(eb) <= 1e-4
        assert int(e) > 0 and int(v) > 0
    # the batch's own hop is the last layer: 1,024 destinations with at most 25 sampled neighbours each
    assert rows[1][2] == "1024" and int(rows[1][3]) <= 1024 * 25
    assert "worst_max_rel_err" in out


@pytest.mark.parametrize("mode", ["pipeline", "explicit", "zerocopy"])
def test_gcn_gpu_neighbor_toolkit_runs_unchanged(arxiv_shaped_files, mode):
    """The toolkit's three batch loops (toolkits/GCN_GPU_NEIGHBOR.hpp:767-775): `pipeline` (stage threads),
    `explicit` (features gathered on the host, then copied) and `zerocopy` (gathered by the device from
    pinned host memory; this loop also fills the `graph` and `nn` columns of the log line)."""
    d = arxiv_shaped_files
    out = run(NTS, write_cfg(d, "GCNNEIGHBORGPU", MODE=mode), cwd=d)
    epochs = re.findall(r"Epoch (\d+) train_loss (\S+) train_acc (\S+) val_loss (\S+) val_acc (\S+) test_acc (\S+) "
                        r"train_time (\S+)\(sample (\S+) trans (\S+) graph (\S+) nn (\S+)\)", out)
    assert [e[0] for e in epochs] == ["000", "001"]
    for e in epochs:
        print("Epoch %s train_loss %s train_acc %s val_loss %s val_acc %s test_acc %s train_time %s(sample %s trans %s "
              "graph %s nn %s)" % e)
        assert all(math.isfinite(float(x)) for x in e[1:])
        assert 0 < float(e[1]) < 10 and 0 <= float(e[2]) <= 1
    assert float(epochs[1][1]) < float(epochs[0][1])  # the loss moves: gradients reach the weights


def test_gcn_gpu_neighbor_toolkit_with_feature_cache_and_two_pipelines(arxiv_shaped_files):
    """The cached gather (top 20 % by degree in HBM, toolkits/GCN_GPU_NEIGHBOR.hpp:899-967) and the
    PIPELINES mode: two host threads, each with a Cuda_Stream bound to a libtorch pool stream."""
    d = arxiv_shaped_files
    out = run(NTS, write_cfg(d, "GCNNEIGHBORGPU", CACHE_TYPE="rate", CACHE_RATE=0.2, CACHE_POLICY="degree", PIPELINES=2),
              cwd=d)
    epochs = re.findall(r"Epoch (\d+) train_loss (\S+) train_acc (\S+)", out)
    assert [e[0] for e in epochs] == ["000", "001"]
    assert all(math.isfinite(float(e[1])) and 0 < float(e[1]) < 10 for e in epochs)


@pytest.mark.parametrize("algorithm", ["GCNEAGERSINGLE", "GINGPU", "GATGPUDIST"])
def test_full_graph_toolkits_run_unchanged(arxiv_shaped_files, algorithm):
    d = arxiv_shaped_files
    # full-batch steps without dropout: the loss of a working backward pass falls from step to step
    out = run(NTS, write_cfg(d, algorithm, EPOCHS=8, DROP_RATE=0), cwd=d)
    losses = [float(x) for x in re.findall(r"Epoch\[\d+\]:(?:Times\[[^\]]*\]:)?loss\s+(\S+)", out)]
    print(f"{algorithm}: losses {losses}")
    assert len(losses) == 8 and all(math.isfinite(x) and 0 < x < 20 for x in losses)
    assert losses[-1] < losses[0]


@pytest.mark.parametrize("algorithm,extra,expect", [
    ("GCNNEIGHBORGPUEXP3", {}, r"Epoch 001 epoch_time \S+ sample_time \S+ gather_time \S+ trans_time \S+ train_time"),
    ("GCNNEIGHBORGPUCACHEEXP", dict(CACHE_TYPE="rate", CACHE_POLICY="degree", CACHE_RATE_START=0.0, CACHE_RATE_END=0.3,
                                    CACHE_RATE_NUM=3), r"cache_rate 0\.300 cache_hit_rate 0\.\d+"),
    ("GCNNEIGHBORGPUTRANSEXP", dict(MODE="zerocopy", TRANS_THRESHOLD_START=0.0, TRANS_THRESHOLD_END=0.5,
                                    TRANS_THRESHOLD_NUM=2), r"Epoch 001 epoch_time \S+ cache_rate"),
    ("GCNEAGER", {}, r"Epoch\[1\]:loss\s+\S+"),
    ("COMMNETGPU", {}, r"Epoch\[1\]:loss\s+\S+"),
])
def test_further_gpu_toolkits_of_the_reference_run_to_the_end(arxiv_shaped_files, algorithm, extra, expect):
    """The other single-GPU entries of toolkits/main.cpp that reach this library: the experiment variants
    of the sampled GCN (epoch breakdown, feature-cache sweep with the cached gather, transfer-threshold
    sweep), the eager full-graph GCN and CommNet.  They must run to their end and print their epoch lines."""
    d = arxiv_shaped_files
    out = run(NTS, write_cfg(d, algorithm, **extra), cwd=d)
    found = re.findall(expect, out)
    print(f"{algorithm}: {found[-1] if found else None}")
    assert found
    if algorithm == "GCNNEIGHBORGPUCACHEEXP":  # the top 30 % of the vertices by degree serve most of the gathered rows
        assert float(found[-1].split()[-1]) > 0.5
