"""Mini-batch assembly: mirrors of Sampler::load_feature_gpu / load_feature_gpu_cache /
load_label_gpu (core/ntsSampler.hpp:353-529) and of the toolkit's cache set-up
(toolkits/GCN_GPU_NEIGHBOR.hpp:899-967), over the C ABI."""
import ctypes

import torch

from .abi import SampledLayerDesc, call, ptr
from .layout import SampledLayer, as_u32
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
    if E:
        call("nts_sample_hop_neighbors", ptr(ri), ptr(co), ptr(graph_co), ptr(graph_ri), ptr(dst), n, fanout, seed,
             stream)
    return co, ri


class DevArray:
    """A typed range of device memory inside a larger torch allocation: what `ptr()` and the
    operators need (address, device, element count) without creating a tensor per array and batch."""
    __slots__ = ("owner", "address", "count", "dtype")

    def __init__(self, owner, address, count, dtype):
        self.owner, self.address, self.count, self.dtype = owner, address, count, dtype

    def data_ptr(self):
        return self.address

    def numel(self):
        return self.count

    @property
    def device(self):
        return self.owner.device

    def tensor(self):
        start = self.address - self.owner.data_ptr()
        return self.owner[start:start + 4 * self.count].view(self.dtype)

    def cpu(self):
        return self.tensor().cpu()


class BatchBuilder:
    """All layers of a mini-batch built on the device without a host step between the hops
    (nts_batch_builder_*): the whole of Sampler::sample_one's construction for every hop
    (core/ntsSampler.hpp:843-1106), one read-back of the layer shapes per batch.

    graph_co / graph_ri: int32 device tensors (uint32 bit patterns) of the whole graph's CSC;
    fanouts: hop 0 (the batch's own hop) first.  The layers returned by `sample` are views into
    this object's arena: they are overwritten by the next `sample`.  graph=True: the launches of the
    hops are recorded once as a HIP graph and replayed for every later batch (same arrays, less host
    time per batch)."""

    def __init__(self, graph_co, graph_ri, fanouts, max_batch, want_perm=False, graph=False):
        self.device = graph_co.device
        self.graph_co, self.graph_ri = graph_co, graph_ri
        self.hops = len(fanouts)
        V, E = graph_co.numel() - 1, graph_ri.numel()
        fan = (ctypes.c_int32 * self.hops)(*fanouts)
        nbytes = call("nts_batch_builder_arena_bytes", V, E, fan, self.hops, max_batch, int(want_perm))
        if nbytes == 0:
            raise ValueError("nts_batch_builder_arena_bytes: unsupported configuration")
        self.arena = torch.empty(nbytes + 256, dtype=torch.uint8, device=self.device)
        self._skew = (-self.arena.data_ptr()) % 256
        handle = ctypes.c_void_p()
        call("nts_batch_builder_create", ctypes.byref(handle), ptr(graph_co), ptr(graph_ri), V, E, fan, self.hops,
             max_batch, int(want_perm), self.arena.data_ptr() + self._skew, nbytes)
        self.handle = handle.value
        # True/1: one recorded chain of launches; 2: hop transpositions on a side branch; 3: sampling and
        # transpositions as two graphs, the second on a stream of the builder's (see `join`)
        if graph:
            call("nts_batch_builder_use_graph", self.handle, int(graph))
        self._desc = (SampledLayerDesc * self.hops)()

    def _array(self, address, count, dtype):
        return DevArray(self.arena, address, count, dtype) if address else None

    def sample(self, batch_ids, seed):
        """batch_ids: int32 device tensor.  Returns the SampledLayer list, input-side layer first;
        the arrays are DevArray ranges of the arena (`.tensor()` gives a torch view)."""
        self.enqueue(batch_ids, seed)
        return self.collect()

    def enqueue(self, batch_ids, seed, stream=None):
        """Starts building a batch on `stream` (a raw stream handle; default: torch's current one)
        and returns at once; `collect` waits for it.  batch_ids must stay alive until then."""
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        call("nts_batch_builder_sample", self.handle, ptr(batch_ids), batch_ids.numel(), seed, stream)

    def join(self, stream=None):
        """Makes `stream` (a raw handle; default: torch's current stream) wait on the device for every
        array of the current batch; only a builder created with graph=3 has anything to wait for."""
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        call("nts_batch_builder_join", self.handle, stream)

    def collect(self, join=True):
        """Waits for the batch started by `enqueue`.  The layers are complete when this returns --
        for a builder created with graph=3: complete for work enqueued on torch's current stream
        (join=True), or, with join=False, only the sampled half (destination, source, column_offset,
        row_indices; the caller calls `join` before the first use of the other arrays)."""
        call("nts_batch_builder_layers", self.handle, ctypes.addressof(self._desc))
        if join:
            self.join()
        layers = []
        i32, f32 = torch.int32, torch.float32
        for d in self._desc:
            layer = SampledLayer()
            Vd, E, Vs = d.v_size, d.e_size, d.src_size
            layer.v_size, layer.e_size, layer.src_size = Vd, E, Vs
            layer.max_in_degree = d.max_in_degree
            layer.dev_destination = self._array(d.destination, Vd, i32)
            layer.dev_source = self._array(d.source, Vs, i32)
            layer.dev_column_offset = self._array(d.column_offset, Vd + 1, i32)
            layer.dev_row_indices = self._array(d.row_indices, E, i32)
            layer.dev_row_offset = self._array(d.row_offset, Vs + 1, i32)
            layer.dev_column_indices = self._array(d.column_indices, E, i32)
            layer.dev_csr_to_csc = self._array(d.csr_to_csc, E, i32)
            layer.dev_edge_weight_forward = self._array(d.edge_weight_forward, E, f32)
            layer.dev_edge_weight_backward = self._array(d.edge_weight_backward, E, f32)
            layers.append(layer)
        return layers

    def close(self):
        if self.handle:
            call("nts_batch_builder_destroy", self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
