"""Drop-in check of the C++ boundary: the reference's own GPU-side headers (full-graph fused op,
the GPU edge operators, NtsScheduler, GraphSegment, sampCSC, FullyRepGraph, the data loader) and
core/GraphSegment.cpp are compiled (syntax only) with CUDA_ENABLE=1 against
neutronbench_amd/host/ntsHIP.hpp through the forwarding headers in neutronbench_amd/host/compat.
Needs the reference tree, so it only runs where /root/reference exists; never on the GPU box.
core/ntsMiniBatchGraphOp.hpp and the toolkits cannot be checked: they include METIS headers that
the tree does not carry."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not present")


def _includes():
    import torch

    t = os.path.join(os.path.dirname(torch.__file__), "include")
    dirs = [os.path.join(ROOT, "neutronbench_amd", "host", "compat"), os.path.join(ROOT, "include"), REF,
            os.path.join(REF, "core"), os.path.join(REF, "comm"), os.path.join(REF, "dep", "gemini"),
            os.path.join(REF, "utils"), "/opt/conda/include", t, os.path.join(t, "torch", "csrc", "api", "include")]
    return [f"-I{d}" for d in dirs]


@pytest.mark.parametrize("source", [os.path.join(ROOT, "tests", "cpp", "reference_gpu_ops_tu.cpp"),
                                    os.path.join(REF, "core", "GraphSegment.cpp")])
def test_reference_sources_parse_against_the_veneer(source):
    if not os.path.exists("/opt/conda/include/mpi.h"):
        pytest.skip("MPI headers not present")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-fopenmp", "-w", "-DCUDA_ENABLE=1", source] + _includes()
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    errors = [line for line in r.stderr.splitlines() if "error" in line]
    assert r.returncode == 0, "\n".join(errors[:20])
