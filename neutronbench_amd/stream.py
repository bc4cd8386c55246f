"""``CudaStream``: Python mirror of the reference's ``Cuda_Stream`` class (cuda/ntsCUDA.hpp:99-211)
over the C ABI, with the reference's method names and argument order.  Arguments are torch tensors
(or raw integer addresses); sizes keep the reference's meaning.  The unused range arguments
(src_end, dst_end) are accepted and ignored exactly as the reference's kernels ignore them.

By default the object wraps torch's current HIP stream of the given device, the way the toolkits
bind a Cuda_Stream to a torch pool stream (toolkits/GCN_GPU_NEIGHBOR.hpp:1350-1363), so graph
kernels and torch work are ordered on one stream.
"""
import torch

from . import abi
from .abi import call, ptr


class CudaStream:
    def __init__(self, stream=None, device=0, synchronize=True):
        """synchronize=False: the batch-assembly methods, which in the reference end with a
        cudaStreamSynchronize, only enqueue their work; for a caller that overlaps the gather of one
        batch with the training of another and orders them with events."""
        if stream is None:
            stream = torch.cuda.current_stream(device).cuda_stream
        self.stream = int(stream)
        self.synchronize = bool(synchronize)

    # -- stream plumbing ----------------------------------------------------------------------
    def getStream(self):
        return self.stream

    def setNewStream(self, stream):
        self.stream = int(stream)

    def CUDA_DEVICE_SYNCHRONIZE(self):
        call("nts_stream_sync", self.stream)

    def _end_of_method(self):
        if self.synchronize:
            self.CUDA_DEVICE_SYNCHRONIZE()

    # -- aggregation --------------------------------------------------------------------------
    def Gather_By_Dst_From_Src(self, input, output, weight_forward, row_indices, column_offset, src_start, src_end,
                               dst_start, dst_end, edges, batch_size, feature_size, with_weight=False,
                               tensor_weight=False):
        """output[d,:] += sum_{e in CSC(d)} w[e] * input[row_indices[e] - src_start, :] (reference
        semantics: accumulates into a pre-zeroed output)."""
        if with_weight and tensor_weight:
            raise abi.NtsError("Gather_By_Dst_From_Src", abi.NTS_ERR_UNSUPPORTED, "tensor weights are a legacy path")
        call("nts_spmm_gather", ptr(input), ptr(output), ptr(weight_forward) if with_weight else 0,
             ptr(column_offset), ptr(row_indices), src_start, batch_size, edges, feature_size, 1, self.stream)

    Gather_By_Dst_From_Src_Optim = Gather_By_Dst_From_Src

    def Gather_By_Src_From_Dst(self, input, output, weight_backward, row_offset, column_indices, src_start, src_end,
                               dst_start, dst_end, edges, batch_size, feature_size, with_weight=False,
                               tensor_weight=False):
        """output[s,:] += sum_{e in CSR(s)} w[e] * input[column_indices[e] - dst_start, :]."""
        if with_weight and tensor_weight:
            raise abi.NtsError("Gather_By_Src_From_Dst", abi.NTS_ERR_UNSUPPORTED, "tensor weights are a legacy path")
        call("nts_spmm_gather", ptr(input), ptr(output), ptr(weight_backward) if with_weight else 0,
             ptr(row_offset), ptr(column_indices), dst_start, batch_size, edges, feature_size, 1, self.stream)

    Gather_By_Src_From_Dst_Optim = Gather_By_Src_From_Dst

    def Scatter_Grad_Back_To_Message(self, input, message_grad, row_indices, column_offset, src_start, src_end,
                                     dst_start, dst_end, edges, batch_size, feature_size, with_weight=True):
        if with_weight:
            raise abi.NtsError("Scatter_Grad_Back_To_Message", abi.NTS_ERR_UNSUPPORTED,
                               "tensor_weight Scatter_Grad_Back_To_Weight not implemented")
        call("nts_scatter_grad_to_edge", ptr(message_grad), ptr(input), ptr(column_offset), batch_size, feature_size,
             self.stream)

    # -- edge ops -----------------------------------------------------------------------------
    def Scatter_Src_Mirror_to_Msg(self, message, src_mirror_feature, row_indices, column_offset, mirror_index,
                                  batch_size, feature_size):
        call("nts_scatter_src_to_edge", ptr(message), ptr(src_mirror_feature), ptr(row_indices), ptr(column_offset),
             ptr(mirror_index), batch_size, feature_size, self.stream)

    def Scatter_Dst_to_Msg(self, message, dst_feature, row_indices, column_offset, batch_size, feature_size):
        call("nts_scatter_dst_to_edge", ptr(message), ptr(dst_feature), ptr(column_offset), batch_size, feature_size,
             self.stream)

    def Gather_Msg_to_Dst(self, dst_feature, message, row_indices, column_offset, batch_size, feature_size):
        call("nts_gather_edge_to_dst", ptr(dst_feature), ptr(message), ptr(column_offset), batch_size, feature_size, 1,
             self.stream)

    def Gather_Msg_To_Src_Mirror(self, src_mirror_feature, message, row_offset, csr_to_csc, src_size, feature_size):
        """Deterministic form: needs the transposed structure (row_offset, csr_to_csc permutation)
        instead of the reference's (row_indices, column_offset, mirror_index) + float atomics."""
        call("nts_gather_edge_to_src", ptr(src_mirror_feature), ptr(message), ptr(row_offset), ptr(csr_to_csc),
             src_size, feature_size, 1, self.stream)

    def Edge_Softmax_Forward_Block(self, msg_output, msg_input, msg_cached, row_indices, column_offset, batch_size,
                                   feature_size):
        call("nts_edge_softmax_fwd", ptr(msg_output), ptr(msg_input), ptr(column_offset), batch_size, feature_size,
             self.stream)
        if msg_cached is not None and ptr(msg_cached) != ptr(msg_output):
            msg_cached.copy_(msg_output)

    def Edge_Softmax_Backward_Block(self, msg_input_grad, msg_output_grad, msg_cached, row_indices, column_offset,
                                    batch_size, feature_size):
        call("nts_edge_softmax_bwd", ptr(msg_input_grad), ptr(msg_output_grad), ptr(msg_cached), ptr(column_offset),
             batch_size, feature_size, self.stream)

    # -- batch assembly -----------------------------------------------------------------------
    def zero_copy_feature_move_gpu(self, dev_feature, pinned_host_feature, src_vertex, feature_size, vertex_size):
        call("nts_gather_rows_f32", ptr(dev_feature), ptr(pinned_host_feature), ptr(src_vertex), 0, 0, vertex_size,
             feature_size, self.stream)
        self._end_of_method()

    def zero_copy_feature_move_gpu_cache(self, dev_feature, pinned_host_feature, src_vertex, feature_size,
                                         vertex_size, local_idx):
        call("nts_gather_rows_f32", ptr(dev_feature), ptr(pinned_host_feature), ptr(src_vertex), ptr(local_idx), 0,
             vertex_size, feature_size, self.stream)
        self._end_of_method()

    def gather_feature_from_gpu_cache(self, dev_feature, dev_cache_feature, src_vertex, feature_size, vertex_size,
                                      local_idx_cache, cache_node_hashmap):
        call("nts_gather_rows_f32", ptr(dev_feature), ptr(dev_cache_feature), ptr(src_vertex), ptr(local_idx_cache),
             ptr(cache_node_hashmap), vertex_size, feature_size, self.stream)
        self._end_of_method()

    def global_copy_label_move_gpu(self, dev_label, global_dev_label, dst_vertex, vertex_size):
        call("nts_gather_labels_i64", ptr(dev_label), ptr(global_dev_label), ptr(dst_vertex), vertex_size, 1,
             self.stream)
        self._end_of_method()

    def global_copy_mulilabel_move_gpu(self, dev_label, global_dev_label, dst_vertex, vertex_size, label_size):
        call("nts_gather_labels_i64", ptr(dev_label), ptr(global_dev_label), ptr(dst_vertex), vertex_size, label_size,
             self.stream)
        self._end_of_method()


def get_gpu_mem():
    """(used, total) device memory in MiB, like utils/cuda_memory.hpp:get_gpu_mem."""
    import ctypes

    free_b = ctypes.c_size_t()
    total_b = ctypes.c_size_t()
    call("nts_mem_info", ctypes.byref(free_b), ctypes.byref(total_b))
    return (total_b.value - free_b.value) / 1048576.0, total_b.value / 1048576.0
