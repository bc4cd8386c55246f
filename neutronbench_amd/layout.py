"""Device-resident graph structure: the full-graph chunk (CSC_segment_pinned's device fields,
core/GraphSegment.h:54-133) and the sampled layer (sampCSC's dev_* arrays, core/coocsc.hpp:806-813).

HBM layout.  Offsets and indices are uint32, weights fp32, each array contiguous:
  column_offset [V_d+1] | row_indices [E] | edge_weight_forward [E]      (CSC, forward)
  row_offset    [V_s+1] | column_indices [E] | edge_weight_backward [E]  (CSR, backward)
torch has no uint32 arithmetic, so tensors are stored as int32 with the same bit pattern; the
kernels read them as uint32.
"""
import ctypes
import time

import torch

from .abi import call, ptr


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def as_u32(t):
    """int64 tensor of values < 2^32 -> int32 tensor with the uint32 bit pattern."""
    return (t & 0xFFFFFFFF).to(torch.int64).add_(1 << 31).remainder_(1 << 32).sub_(1 << 31).to(torch.int32)


def u32_to_i64(t):
    return t.to(torch.int64) & 0xFFFFFFFF


class SpmmPlan:
    """Degree-bucketed schedule bound to one offsets tensor."""

    def __init__(self, offsets, rows, edges, chunk_edges=0, indices=None, n_index=0, n_slabs=0):
        """indices / n_index given: cache-aware schedule (split rows cut at source-range boundaries
        and issued range by range); otherwise split rows are cut every chunk_edges edges."""
        self.offsets = offsets
        handle = ctypes.c_void_p()
        if indices is not None:
            call("nts_spmm_plan_create_slabs", ctypes.byref(handle), ptr(offsets), ptr(indices), 0, n_index, rows,
                 edges, chunk_edges, n_slabs, _stream(offsets.device))
        else:
            call("nts_spmm_plan_create", ctypes.byref(handle), ptr(offsets), rows, edges, chunk_edges,
                 _stream(offsets.device))
        self.handle = handle.value

    def info(self):
        a, b, c = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
        call("nts_spmm_plan_info", self.handle, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
        return dict(items=a.value, split_rows=b.value, partials=c.value)

    def reserve(self, F):
        call("nts_spmm_plan_reserve", self.handle, F)

    def scratch_info(self, F):
        """Scratch a call of width F keeps in the plan and what the schedule found about parallel edges."""
        pb, ib, rep, runs = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_uint64(), ctypes.c_int()
        call("nts_spmm_plan_scratch_info", self.handle, F, ctypes.byref(pb), ctypes.byref(ib), ctypes.byref(rep),
             ctypes.byref(runs))
        return dict(partial_bytes=pb.value, padded_input_bytes=ib.value, repeated_edges=rep.value,
                    loads_once_per_run=bool(runs.value))

    def close(self):
        if self.handle:
            call("nts_spmm_plan_destroy", self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class FullGraphChunk:
    """One partition's CSC + CSR + GCN weights in HBM, plus the aggregation schedules."""

    def __init__(self, V, column_offset, row_indices, ewf, row_offset, column_indices, ewb, chunk_edges=0, n_slabs=1):
        self.V = V
        self.E = int(row_indices.numel())
        self.column_offset_gpu = column_offset
        self.row_indices_gpu = row_indices
        self.edge_weight_forward_gpu = ewf
        self.row_offset_gpu = row_offset
        self.column_indices_gpu = column_indices
        self.edge_weight_backward_gpu = ewb
        self.src_range = (0, V)
        self.dst_range = (0, V)
        torch.cuda.current_stream(column_offset.device).synchronize()
        t0 = time.perf_counter()
        if n_slabs == 1:
            self.plan_forward = SpmmPlan(column_offset, V, self.E, chunk_edges)
            self.plan_backward = SpmmPlan(row_offset, V, self.E, chunk_edges)
        else:
            self.plan_forward = SpmmPlan(column_offset, V, self.E, chunk_edges, row_indices, V, n_slabs)
            self.plan_backward = SpmmPlan(row_offset, V, self.E, chunk_edges, column_indices, V, n_slabs)
        self.plan_build_s = time.perf_counter() - t0  # both schedules (host side, read-backs and uploads included)

    @classmethod
    def from_edges(cls, src, dst, V, chunk_edges=0, n_slabs=1):
        """Builds the chunk on the device that holds `src` / `dst` (int64 edge list).

        Edge order follows PartitionToChunks (core/PartitionedGraph.hpp:281-388): the COO list is
        ordered by source (stable in the input order); CSR rows keep that order, CSC rows are the
        stable re-ordering by destination.  Weights are nts_norm_degree of the global degrees.
        """
        pairs = torch.stack([src, dst], dim=1).to(torch.int32).contiguous()
        return cls.from_edge_pairs(pairs, V, chunk_edges, n_slabs)

    @classmethod
    def from_edge_pairs(cls, pairs, V, chunk_edges=0, n_slabs=1):
        """`pairs`: int32 device tensor [E, 2] holding the .edge file's records (src, dst)."""
        device = pairs.device
        E = pairs.shape[0]
        co32 = torch.empty(V + 1, dtype=torch.int32, device=device)
        ro32 = torch.empty(V + 1, dtype=torch.int32, device=device)
        ri32 = torch.empty(E, dtype=torch.int32, device=device)
        ci32 = torch.empty(E, dtype=torch.int32, device=device)
        ewf = torch.empty(E, dtype=torch.float32, device=device)
        ewb = torch.empty(E, dtype=torch.float32, device=device)
        work = torch.empty(call("nts_chunk_from_edges_work_bytes", V, E) + 256, dtype=torch.uint8, device=device)
        wptr = (work.data_ptr() + 255) // 256 * 256
        call("nts_chunk_from_edges", ptr(co32), ptr(ri32), ptr(ewf), ptr(ro32), ptr(ci32), ptr(ewb), ptr(pairs), E, V,
             wptr, _stream(device))
        torch.cuda.current_stream(device).synchronize()  # `work` and `pairs` may be released by the caller
        del work
        return cls(V, co32, ri32, ewf, ro32, ci32, ewb, chunk_edges, n_slabs)

    @classmethod
    def from_edge_file(cls, path, V, device, chunk_edges=0, n_slabs=1):
        """Graph::load_directed + PartitionToChunks for one partition: reads the binary edge list
        into pinned memory, uploads it once and builds CSC, CSR and weights on the device."""
        from .dataset import edge_file_count, read_edge_file

        E = edge_file_count(path)
        host = torch.empty((E, 2), dtype=torch.int32, pin_memory=True)
        read_edge_file(path, vertices=V, out=host.numpy().view("uint32"))
        return cls.from_edge_pairs(host.to(device, non_blocking=True), V, chunk_edges, n_slabs)


class SampledLayer:
    """Device mirror of one sampCSC: destination / source (global ids), CSC, CSR, weights.

    `from_host_csc` takes what the sampler's host steps produce (column_offset, local row_indices,
    source, destination) in one packed upload and builds the CSR and both weight arrays on the
    device (generate_csr_from_csc + update_degree + compute_weight_*), replacing the reference's
    eight host-built arrays and eight copies per layer (core/coocsc.hpp:737-773).
    """

    def __init__(self):
        self.v_size = self.e_size = self.src_size = 0
        self.max_in_degree = 0  # bound on a destination's edges where the sampler knows one (its fanout), else 0
        self.dev_destination = self.dev_source = None
        self.dev_column_offset = self.dev_row_indices = None
        self.dev_row_offset = self.dev_column_indices = None
        self.dev_edge_weight_forward = self.dev_edge_weight_backward = None
        self.dev_csr_to_csc = None

    @classmethod
    def from_host_csc(cls, column_offset, row_indices, source, destination, device, want_perm=True):
        self = cls()
        Vd, E, Vs = destination.numel(), row_indices.numel(), source.numel()
        self.v_size, self.e_size, self.src_size = Vd, E, Vs
        packed = torch.cat([as_u32(column_offset), as_u32(row_indices), as_u32(source), as_u32(destination)])
        if device.type == "cuda":
            packed = packed.pin_memory().to(device, non_blocking=True)
        co, ri, src, dst = torch.split(packed, [Vd + 1, E, Vs, Vd])
        self.dev_column_offset, self.dev_row_indices, self.dev_source, self.dev_destination = co, ri, src, dst
        self._finish_on_device(want_perm)
        return self

    @classmethod
    def from_device_hop(cls, column_offset, row_indices_global, destination, V, want_perm=True):
        """Whole construction on the device: `column_offset` [Vd+1] and `row_indices_global` [E]
        (global source ids of the sampled edges) and `destination` [Vd] are int32 device tensors.
        Relabels the sources (sampCSC::postprocessing), then builds the CSR and the weights."""
        self = cls()
        device = column_offset.device
        Vd, E = destination.numel(), row_indices_global.numel()
        stream = _stream(device)
        work_bytes = call("nts_relabel_sources_work_bytes", V)
        work = torch.empty(work_bytes + 256, dtype=torch.uint8, device=device)
        base = (work.data_ptr() + 255) // 256 * 256
        source = torch.empty(max(min(E, V), 1), dtype=torch.int32, device=device)
        n_source = torch.zeros(1, dtype=torch.int32, device=device)
        local = torch.empty(E, dtype=torch.int32, device=device)
        call("nts_relabel_sources", ptr(source), ptr(n_source), ptr(local), ptr(row_indices_global), E, V, base, stream)
        Vs = int(n_source.item())  # the one read-back of the construction: sizes the CSR arrays
        self.v_size, self.e_size, self.src_size = Vd, E, Vs
        self.dev_column_offset, self.dev_row_indices = column_offset, local
        self.dev_source, self.dev_destination = source[:Vs], destination
        self._finish_on_device(want_perm)
        return self

    def _finish_on_device(self, want_perm):
        device = self.dev_column_offset.device
        Vd, E, Vs = self.v_size, self.e_size, self.src_size
        self.dev_row_offset = torch.empty(Vs + 1, dtype=torch.int32, device=device)
        self.dev_column_indices = torch.empty(E, dtype=torch.int32, device=device)
        self.dev_csr_to_csc = torch.empty(E, dtype=torch.int32, device=device) if want_perm else None
        self.dev_edge_weight_forward = torch.empty(E, dtype=torch.float32, device=device)
        self.dev_edge_weight_backward = torch.empty(E, dtype=torch.float32, device=device)
        stream = _stream(device)
        work_bytes = call("nts_csr_from_csc_work_bytes", Vd, Vs, E)
        work = torch.empty(max(work_bytes, 256) + 256, dtype=torch.uint8, device=device)
        base = (work.data_ptr() + 255) // 256 * 256
        call("nts_csr_from_csc", ptr(self.dev_row_offset), ptr(self.dev_column_indices), ptr(self.dev_csr_to_csc),
             ptr(self.dev_column_offset), ptr(self.dev_row_indices), Vd, Vs, E, base, stream)
        call("nts_gcn_edge_weights", ptr(self.dev_edge_weight_forward), ptr(self.dev_edge_weight_backward),
             ptr(self.dev_column_offset), ptr(self.dev_row_indices), ptr(self.dev_row_offset),
             ptr(self.dev_column_indices), Vd, Vs, stream)

    # accessor names of the reference (core/coocsc.hpp: dev_c_o() ... dev_ewb())
    def dev_c_o(self):
        return self.dev_column_offset

    def dev_r_i(self):
        return self.dev_row_indices

    def dev_r_o(self):
        return self.dev_row_offset

    def dev_c_i(self):
        return self.dev_column_indices

    def dev_ewf(self):
        return self.dev_edge_weight_forward

    def dev_ewb(self):
        return self.dev_edge_weight_backward
