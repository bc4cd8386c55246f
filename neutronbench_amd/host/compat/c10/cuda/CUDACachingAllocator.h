// The libtorch names that NeutronBench's GPU toolkits spell (toolkits/GCN_GPU_NEIGHBOR.hpp:1, 86, 461,
// 1247, 1351-1353 and its variants), provided over libtorch's ROCm build so that the toolkits compile
// unchanged: the ROCm build of libtorch ships these facilities under c10::hip with the
// "MasqueradingAsCUDA" stream type (a HIP stream whose device type is the one ROCm tensors carry).
//
//   c10::cuda::CUDACachingAllocator::emptyCache      -> c10::hip::HIPCachingAllocator::emptyCache
//   at::cuda::CUDAStream                             -> c10::hip::HIPStreamMasqueradingAsCUDA
//   at::cuda::getDefaultCUDAStream / setCurrentCUDAStream / getStreamFromPool
//
// getStreamFromPool ignores its priority argument: the toolkit asks for high-priority pool streams
// (GCN_GPU_NEIGHBOR.hpp:1353), and every stream of this build stays at the default priority.
#pragma once

#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPCachingAllocator.h>

namespace c10 {
namespace cuda {

using CUDAStream = c10::hip::HIPStreamMasqueradingAsCUDA;

inline CUDAStream getStreamFromPool(const bool /*isHighPriority*/ = false, DeviceIndex device = -1) {
  return c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, device);
}
inline CUDAStream getDefaultCUDAStream(DeviceIndex device = -1) {
  return c10::hip::getDefaultHIPStreamMasqueradingAsCUDA(device);
}
inline CUDAStream getCurrentCUDAStream(DeviceIndex device = -1) {
  return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device);
}
inline void setCurrentCUDAStream(CUDAStream stream) { c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(stream); }

namespace CUDACachingAllocator {
inline void emptyCache() { c10::hip::HIPCachingAllocator::emptyCache(); }
}  // namespace CUDACachingAllocator

}  // namespace cuda
}  // namespace c10

// Using-declarations, not a using-directive: libtorch's ROCm headers already pull c10::hip into
// at::cuda, and names declared in a namespace itself are found before those a directive nominates.
namespace at {
namespace cuda {
using c10::cuda::CUDAStream;
using c10::cuda::getCurrentCUDAStream;
using c10::cuda::getDefaultCUDAStream;
using c10::cuda::getStreamFromPool;
using c10::cuda::setCurrentCUDAStream;
}  // namespace cuda
}  // namespace at
