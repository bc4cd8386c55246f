// Device-memory queries for the toolkits (replaces utils/cuda_memory.hpp of the NeutronBench tree,
// which sizes the feature cache from the free HBM, toolkits/GCN_GPU_NEIGHBOR.hpp:1427-1441).
// Amounts are MiB, as there.
#ifndef NTS_HIP_MEMORY_HPP
#define NTS_HIP_MEMORY_HPP

#include <stdio.h>

#include <utility>

#include "../../ntsHIP.hpp"

inline void get_gpu_mem(double &used, double &total) {
  size_t free_b = 0, total_b = 0;
  NTS_VENEER_CHECK(nts_mem_info(&free_b, &total_b));
  total = (double)total_b / (1024.0 * 1024.0);
  used = total - (double)free_b / (1024.0 * 1024.0);
}

inline std::pair<double, double> get_gpu_mem() {
  double used = 0, total = 0;
  get_gpu_mem(used, total);
  return {used, total};
}

inline void show_gpu_mem() {
  double used = 0, total = 0;
  get_gpu_mem(used, total);
  printf("used gpu mem %.3fM\n", used);
}

#endif  // NTS_HIP_MEMORY_HPP
