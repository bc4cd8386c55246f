#!/bin/bash
# Builds the reference-derived checkers under oracle/_ref/ from the NeutronBench sources where they
# lie (read-only tree at /root/reference; nothing is copied).  TEST INFRASTRUCTURE ONLY.
#
#   libnts_ref.so       the header-only arithmetic helpers of core/ntsBaseOp.hpp (ref_shim.cpp)
#   ref_fullgraph_cpu   the reference's loader, partitioner and CPU operator classes
#                       (ForwardCPUfuseOp, SingleCPUSrcDstScatterOp, SingleEdgeSoftMax,
#                       SingleCPUDstAggregateOp) behind ref_fullgraph_driver.cpp
#   ref_fullgraph_gpu   the same plus the reference's GPU operator classes (ForwardSingleGPUfuseOp,
#                       DistGPU*), compiled with CUDA_ENABLE=1 against the HIP veneer and linked to
#                       neutronbench_amd/lib/libntship.so (which must have been built before)
#
# The two programs compile core/GraphSegment.cpp and comm/network.cpp from the reference tree and
# link the image's libtorch, MPICH (/opt/conda) and libnuma; nothing else of the reference's build
# is used.  core/ntsMiniBatchGraphOp.hpp and the toolkits need METIS headers the tree does not
# carry and stay unbuilt.  Flags follow the reference's release build (CMakeLists.txt:128: -O3
# -fopenmp, GCC's default floating-point contraction), with -march=x86-64-v3 instead of
# -march=native so that the binaries also run on another host.
#
# libtorch bundles its own libnuma / libgomp under other file names; the two symlinks created
# below make the programs resolve libnuma.so.1 / libgomp.so.1 to those same files, so that only one
# copy of each runtime is loaded.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
ROOT="$(dirname "$HERE")"
REF="${NTS_REFERENCE_DIR:-/root/reference}"
TORCH="$(python3 -c 'import torch, os; print(os.path.dirname(torch.__file__))')"
MPI_DIR="${NTS_MPI_DIR:-/opt/conda}"
OUT="$HERE/_ref"
mkdir -p "$OUT"
CXX="g++ -std=c++17 -O3 -march=x86-64-v3 -fopenmp -w"
REF_INC="-I$REF -I$REF/core -I$REF/comm -I$REF/dep/gemini -I$REF/utils -I$MPI_DIR/include -I$TORCH/include -I$TORCH/include/torch/csrc/api/include"

$CXX -fPIC -shared -fvisibility=hidden -o "$OUT/libnts_ref.so" "$HERE/ref_shim.cpp" -I"$REF/cuda" $REF_INC
echo "built $OUT/libnts_ref.so"

if [ ! -f "$MPI_DIR/include/mpi.h" ] || [ ! -f "$MPI_DIR/lib/libmpi.so" ] || [ ! -f /usr/include/numa.h ]; then
  echo "MPI or libnuma not present: reference operator programs not built"
  exit 0
fi

VENEER_INC="-I$ROOT/neutronbench_amd/host/compat -I$ROOT/include -I/opt/rocm/include"
pids=()
$CXX -DCUDA_ENABLE=0 -c "$HERE/ref_fullgraph_driver.cpp" -o "$OUT/drv_cpu.o" $REF_INC & pids+=($!)
$CXX -DCUDA_ENABLE=0 -c "$REF/core/GraphSegment.cpp" -o "$OUT/seg_cpu.o" $REF_INC & pids+=($!)
$CXX -DCUDA_ENABLE=0 -c "$REF/comm/network.cpp" -o "$OUT/net_cpu.o" $REF_INC & pids+=($!)
$CXX -DCUDA_ENABLE=1 -D__HIP_PLATFORM_AMD__ -c "$HERE/ref_fullgraph_driver.cpp" -o "$OUT/drv_gpu.o" $VENEER_INC $REF_INC & pids+=($!)
$CXX -DCUDA_ENABLE=1 -D__HIP_PLATFORM_AMD__ -c "$REF/core/GraphSegment.cpp" -o "$OUT/seg_gpu.o" $VENEER_INC $REF_INC & pids+=($!)
$CXX -DCUDA_ENABLE=1 -D__HIP_PLATFORM_AMD__ -c "$REF/comm/network.cpp" -o "$OUT/net_gpu.o" $VENEER_INC $REF_INC & pids+=($!)
for p in "${pids[@]}"; do wait "$p"; done

ln -sf "$TORCH/lib/libnuma.so" "$OUT/libnuma.so.1"
ln -sf "$TORCH/lib/libgomp.so" "$OUT/libgomp.so.1"
# Search order at run time: the symlinks, libntship, libtorch, the system's libstdc++ (newer than the
# one under /opt/conda/lib, which only serves libmpi and its own dependencies).
RPATHS="-Wl,-rpath,\$ORIGIN -Wl,-rpath,\$ORIGIN/../../neutronbench_amd/lib -Wl,-rpath,$TORCH/lib -Wl,-rpath,/usr/lib/x86_64-linux-gnu -Wl,-rpath,$MPI_DIR/lib"
g++ -fopenmp -o "$OUT/ref_fullgraph_cpu" "$OUT/drv_cpu.o" "$OUT/seg_cpu.o" "$OUT/net_cpu.o" \
    -L"$TORCH/lib" -ltorch_cpu -lc10 "$MPI_DIR/lib/libmpi.so" -lnuma $RPATHS
echo "built $OUT/ref_fullgraph_cpu"
if [ -f "$ROOT/neutronbench_amd/lib/libntship.so" ]; then
  g++ -fopenmp -o "$OUT/ref_fullgraph_gpu" "$OUT/drv_gpu.o" "$OUT/seg_gpu.o" "$OUT/net_gpu.o" \
      -L"$TORCH/lib" -ltorch -ltorch_cpu -ltorch_hip -lc10 -lc10_hip -L"$ROOT/neutronbench_amd/lib" -lntship \
      "$MPI_DIR/lib/libmpi.so" -lnuma $RPATHS
  echo "built $OUT/ref_fullgraph_gpu"
else
  echo "neutronbench_amd/lib/libntship.so missing: ref_fullgraph_gpu not built"
fi
rm -f "$OUT"/*.o
