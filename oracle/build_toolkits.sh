#!/bin/bash
# Builds the reference's own toolkit program (toolkits/main.cpp: GCN_GPU_NEIGHBOR, GIN_GPU,
# GCN_EAGER_single, GAT_GPU_DIST, ... selected by the ALGORITHM line of a .cfg file) from the reference
# tree where it lies, UNCHANGED, against this repository's host veneer and HIP library in place of
# the reference's cuda/ directory:   oracle/_ref/nts
# and, with the same flags and include path, oracle/_ref/ref_minibatch (ref_minibatch_driver.cpp: the
# reference's sampler, MiniBatchFuseOp and SingleGPUSampleGraphOp on the same sampled layers).
#
# This is the swap a maintainer makes (the reference's CMake target `nts`, CMakeLists.txt:136-153,
# with cuda_propagate replaced by libntship.so and ${TORCH_LIBRARIES} by libtorch's ROCm build),
# spelled as plain g++ commands because the reference's CMake files insist on nvcc and on the METIS
# submodule.  Same sources (toolkits/main.cpp, core/GraphSegment.cpp, comm/network.cpp), same
# definitions (CUDA_ENABLE, IDXTYPEWIDTH=64, REALTYPEWIDTH=32), same flags (-O3 -fopenmp; x86-64-v3
# instead of -march=native so that the binary also runs on another host).
#
# METIS: the tree's third_party/METIS submodule is empty.  core/MetisPartition.hpp only needs the
# header's types and two entry points, reached by no configuration run here (BATCH_TYPE metis);
# oracle/toolkit_shims/metis.h declares them for this build alone.  The program is an integration
# demonstration (tests/test_reference_toolkits.py); nothing it prints pins the oracle.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
ROOT="$(dirname "$HERE")"
REF="${NTS_REFERENCE_DIR:-/root/reference}"
TORCH="$(python3 -c 'import torch, os; print(os.path.dirname(torch.__file__))')"
MPI_DIR="${NTS_MPI_DIR:-/opt/conda}"
OUT="$HERE/_ref"
mkdir -p "$OUT"
if [ ! -f "$ROOT/neutronbench_amd/lib/libntship.so" ]; then
  echo "neutronbench_amd/lib/libntship.so missing: build it first (make -C neutronbench_amd/csrc)"; exit 1
fi
if [ ! -f "$MPI_DIR/include/mpi.h" ] || [ ! -f /usr/include/numa.h ]; then
  echo "MPI or libnuma not present: toolkit program not built"; exit 0
fi
CXX="g++ -std=c++17 -O3 -march=x86-64-v3 -fopenmp -w -DCUDA_ENABLE=1 -D__HIP_PLATFORM_AMD__ -DIDXTYPEWIDTH=64 -DREALTYPEWIDTH=32"
INC="-I$HERE/toolkit_shims -I$ROOT/neutronbench_amd/host/compat -I$ROOT/include -I/opt/rocm/include \
     -I$REF -I$REF/core -I$REF/comm -I$REF/cuda -I$REF/dep/gemini -I$REF/utils -I$REF/toolkits \
     -I$MPI_DIR/include -I$TORCH/include -I$TORCH/include/torch/csrc/api/include"
pids=()
$CXX -c "$REF/toolkits/main.cpp" -o "$OUT/tk_main.o" $INC & pids+=($!)
$CXX -c "$REF/core/GraphSegment.cpp" -o "$OUT/tk_seg.o" $INC & pids+=($!)
$CXX -c "$REF/comm/network.cpp" -o "$OUT/tk_net.o" $INC & pids+=($!)
$CXX -c "$HERE/ref_minibatch_driver.cpp" -o "$OUT/tk_mini.o" $INC & pids+=($!)
for p in "${pids[@]}"; do wait "$p"; done
ln -sf "$TORCH/lib/libnuma.so" "$OUT/libnuma.so.1"
ln -sf "$TORCH/lib/libgomp.so" "$OUT/libgomp.so.1"
RPATHS="-Wl,-rpath,\$ORIGIN -Wl,-rpath,\$ORIGIN/../../neutronbench_amd/lib -Wl,-rpath,$TORCH/lib -Wl,-rpath,/usr/lib/x86_64-linux-gnu -Wl,-rpath,$MPI_DIR/lib"
g++ -fopenmp -o "$OUT/nts" "$OUT/tk_main.o" "$OUT/tk_seg.o" "$OUT/tk_net.o" \
    -L"$TORCH/lib" -ltorch -ltorch_cpu -ltorch_hip -lc10 -lc10_hip -L"$ROOT/neutronbench_amd/lib" -lntship \
    "$MPI_DIR/lib/libmpi.so" -lnuma $RPATHS
echo "built $OUT/nts"
# The reference's sampler and both of its mini-batch operator classes behind ref_minibatch_driver.cpp.
g++ -fopenmp -o "$OUT/ref_minibatch" "$OUT/tk_mini.o" "$OUT/tk_seg.o" "$OUT/tk_net.o" \
    -L"$TORCH/lib" -ltorch -ltorch_cpu -ltorch_hip -lc10 -lc10_hip -L"$ROOT/neutronbench_amd/lib" -lntship \
    "$MPI_DIR/lib/libmpi.so" -lnuma $RPATHS
rm -f "$OUT"/tk_*.o
echo "built $OUT/ref_minibatch"
