"""Mini-batch assembly: mirrors of Sampler::load_feature_gpu / load_feature_gpu_cache /
load_label_gpu (core/ntsSampler.hpp:353-529) and of the toolkit's cache set-up
(toolkits/GCN_GPU_NEIGHBOR.hpp:899-967), over the C ABI."""
import ctypes

import torch

from .abi import call, ptr
from .layout import as_u32
from .stream import CudaStream


class MappedHostTable:
    """Feature table in page-locked host memory mapped into the device address space
    (cudaMallocPinned + getDevicePointer of the reference): kernels read it over PCIe."""

    def __init__(self, features):
        n, F = features.shape
        self.shape = (n, F)
        nbytes = n * F * 4
        host = ctypes.c_void_p()
        call("nts_malloc_pinned_mapped", ctypes.byref(host), nbytes)
        self.host_ptr = host.value
        ctypes.memmove(self.host_ptr, features.contiguous().data_ptr(), nbytes)
        dev = ctypes.c_void_p()
        call("nts_host_get_device_ptr", ctypes.byref(dev), self.host_ptr)
        self.dev_ptr = dev.value

    def close(self):
        if self.host_ptr:
            call("nts_free_pinned", self.host_ptr)
            self.host_ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class FeatureCache:
    """HBM cache of the highest out-degree nodes' feature rows; slot = rank in the degree order."""

    def __init__(self, features_cpu, out_degree, n_cache, device):
        V = features_cpu.shape[0]
        # Descending out-degree, ties by ascending id (the reference's std::sort leaves ties unspecified).
        order = torch.sort(out_degree.to(torch.int64), descending=True, stable=True).indices[:n_cache]
        hashmap = torch.full((V,), 0xFFFFFFFF, dtype=torch.int64)
        hashmap[order] = torch.arange(n_cache, dtype=torch.int64)
        self.order = order
        self.n_cache = n_cache
        self.cache_node_hashmap = as_u32(hashmap)
        self.dev_cache_node_hashmap = self.cache_node_hashmap.to(device)
        self.dev_cache_feature = features_cpu[order].contiguous().to(device)


def load_feature_gpu(cs, layer0, local_feature, table_ptr):
    """X0[i,:] = feature[source[i],:] read zero-copy from mapped host memory (or from HBM)."""
    cs.zero_copy_feature_move_gpu(local_feature, table_ptr, layer0.dev_source, local_feature.shape[1],
                                  layer0.src_size)


def load_feature_gpu_cache(cs, layer0, local_feature, table_ptr, cache, source_cpu=None, device_split=True):
    """Cached gather.  device_split=True: one kernel decides hit / miss per row on the device.
    device_split=False: the reference's flow -- host loop builds the two position lists, then one
    launch per list."""
    F = local_feature.shape[1]
    n = layer0.src_size
    if device_split:
        hits = torch.zeros(1, dtype=torch.int32, device=local_feature.device)
        call("nts_gather_rows_cached_f32", ptr(local_feature), table_ptr, ptr(cache.dev_cache_feature),
             ptr(layer0.dev_source), ptr(cache.dev_cache_node_hashmap), n, F, ptr(hits), cs.stream)
        return hits
    slots = cache.cache_node_hashmap[source_cpu.to(torch.int64)]
    hit_pos = torch.nonzero(slots != -1).flatten()
    miss_pos = torch.nonzero(slots == -1).flatten()
    dev = local_feature.device
    d_hit, d_miss = as_u32(hit_pos).to(dev), as_u32(miss_pos).to(dev)
    cs.zero_copy_feature_move_gpu_cache(local_feature, table_ptr, layer0.dev_source, F, miss_pos.numel(), d_miss)
    cs.gather_feature_from_gpu_cache(local_feature, cache.dev_cache_feature, layer0.dev_source, F, hit_pos.numel(),
                                     d_hit, cache.dev_cache_node_hashmap)
    return hit_pos.numel()


def load_label_gpu(cs, top_layer, local_label, global_label):
    classes = 1 if global_label.dim() == 1 else global_label.shape[1]
    if classes > 1:
        cs.global_copy_mulilabel_move_gpu(local_label, global_label, top_layer.dev_destination, top_layer.v_size,
                                          classes)
    else:
        cs.global_copy_label_move_gpu(local_label, global_label, top_layer.dev_destination, top_layer.v_size)


def sample_hop(graph_co, graph_ri, dst, fanout, seed):
    """One hop of neighbour sampling on the device through the library: returns
    (column_offset [n+1], row_indices with GLOBAL source ids [E]) as int32 device tensors.
    graph_co / graph_ri / dst are int32 device tensors (uint32 bit patterns)."""
    device = dst.device
    n = dst.numel()
    stream = torch.cuda.current_stream(device).cuda_stream
    work = torch.empty(call("nts_sample_hop_work_bytes", n) + 256, dtype=torch.uint8, device=device)
    base = (work.data_ptr() + 255) // 256 * 256
    co = torch.empty(n + 1, dtype=torch.int32, device=device)
    call("nts_sample_hop_offsets", ptr(co), ptr(graph_co), ptr(dst), n, fanout, base, stream)
    E = int(co[-1].item()) & 0xFFFFFFFF  # one read-back: sizes the edge array
    ri = torch.empty(E, dtype=torch.int32, device=device)
    call("nts_sample_hop_neighbors", ptr(ri), ptr(co), ptr(graph_co), ptr(graph_ri), ptr(dst), n, fanout, seed, stream)
    return co, ri
