// Exposes a few arithmetic helpers of the NeutronBench sources themselves (compiled from where
// they lie under /root/reference, never copied) behind a C interface, so that the oracle's
// restatement can be validated against the real code.  TEST INFRASTRUCTURE ONLY.
//
//   nts::op::nts_comp, nts::op::dot_product, nts::op::nts_copy   core/ntsBaseOp.hpp:61-97, 167-175
//   nts::op::nts_norm_degree                                     core/ntsBaseOp.hpp:183-186
//
// nts_norm_degree reads two fields of a Graph<Empty>; the graph object here is zero-filled storage
// with only those two array pointers set (constructing a real Graph needs the whole MPI / NUMA
// engine and an edge file).
#include <stdint.h>
#include <stdlib.h>

#include "comm/logger.h"
#include "core/ntsBaseOp.hpp"

extern "C" {

__attribute__((visibility("default"))) void ref_nts_comp(float *output, float *input, float weight, int feat_size) {
  nts::op::nts_comp(output, input, weight, feat_size);
}

__attribute__((visibility("default"))) void ref_nts_comp_non_avx256(float *output, float *input, float weight,
                                                                   int feat_size) {
  nts::op::nts_comp_non_avx256(output, input, weight, feat_size);
}

__attribute__((visibility("default"))) float ref_dot_product(float *a, float *b, int feat_size) {
  return nts::op::dot_product(a, b, feat_size);
}

__attribute__((visibility("default"))) void ref_nts_copy(float *b_dst, long d_offset, float *b_src, uint32_t s_offset,
                                                        int feat_size, int counts) {
  nts::op::nts_copy(b_dst, d_offset, b_src, s_offset, feat_size, counts);
}

__attribute__((visibility("default"))) float ref_nts_norm_degree(uint32_t *out_degree, uint32_t *in_degree,
                                                                uint32_t src, uint32_t dst) {
  static Graph<Empty> *g = nullptr;
  if (!g) g = static_cast<Graph<Empty> *>(calloc(1, sizeof(Graph<Empty>)));
  g->out_degree_for_backward = out_degree;
  g->in_degree_for_backward = in_degree;
  return nts::op::nts_norm_degree(g, src, dst);
}

}  // extern "C"
