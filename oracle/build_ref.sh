#!/bin/bash
# Builds oracle/_ref/libnts_ref.so from the NeutronBench sources where they lie (read-only tree at
# /root/reference; nothing is copied).  Only the header-only arithmetic helpers of
# core/ntsBaseOp.hpp are reachable this way: the CPU operators themselves need the Gemini graph
# engine, an MPI runtime and an edge file, and core/ntsMiniBatchGraphOp.hpp needs METIS headers
# the tree does not carry -- those stay unbuilt and the oracle is pinned without them.
# Flags follow the reference's release build (CMakeLists.txt:128: -O3 -fopenmp with GCC's default
# floating-point contraction), except -march=x86-64-v3 instead of -march=native so that the library
# also runs on another host.  TEST INFRASTRUCTURE ONLY.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
REF="${NTS_REFERENCE_DIR:-/root/reference}"
TORCH="$(python3 -c 'import torch, os; print(os.path.dirname(torch.__file__))')"
MPI_INC="${NTS_MPI_INCLUDE:-/opt/conda/include}"
mkdir -p "$HERE/_ref"
g++ -std=c++17 -O3 -march=x86-64-v3 -fopenmp -fPIC -shared -w -fvisibility=hidden \
    -o "$HERE/_ref/libnts_ref.so" "$HERE/ref_shim.cpp" \
    -I"$REF" -I"$REF/core" -I"$REF/comm" -I"$REF/cuda" -I"$REF/dep/gemini" -I"$REF/utils" \
    -I"$MPI_INC" -I"$TORCH/include" -I"$TORCH/include/torch/csrc/api/include"
echo "built $HERE/_ref/libnts_ref.so"
