"""ctypes binding of libntship.so (include/nts_hip.h).

Pointers are passed as integers: ``ptr(tensor)`` returns ``tensor.data_ptr()`` for a torch tensor,
0 for None and the value itself for an int.  Status codes other than NTS_OK raise ``NtsError`` with
the library's error text.  Loading fails loudly when the library has not been built -- there is no
fallback implementation.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libntship.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

NTS_OK, NTS_ERR_INVALID, NTS_ERR_HIP, NTS_ERR_UNSUPPORTED, NTS_ERR_NOMEM = range(5)

_vp = ctypes.c_void_p
_u32 = ctypes.c_uint32
_int = ctypes.c_int
_sz = ctypes.c_size_t
_f32 = ctypes.c_float
_u64 = ctypes.c_uint64
_str = ctypes.c_char_p

# name -> argument types, in the order of include/nts_hip.h.  All return int unless listed in _RESTYPES.
SIGNATURES = {
    "nts_last_error": [],
    "nts_abi_version": [],
    "nts_trace_ranges_emitted": [],
    "nts_scratch_trim": [],
    "nts_scratch_alloc_count": [],
    "nts_malloc_device": [ctypes.POINTER(_vp), _sz],
    "nts_free_device": [_vp],
    "nts_malloc_device_async": [ctypes.POINTER(_vp), _sz, _vp],
    "nts_free_device_async": [_vp, _vp],
    "nts_malloc_pinned_mapped": [ctypes.POINTER(_vp), _sz],
    "nts_free_pinned": [_vp],
    "nts_host_get_device_ptr": [ctypes.POINTER(_vp), _vp],
    "nts_memcpy_h2d": [_vp, _vp, _sz, _int],
    "nts_memcpy_h2d_async": [_vp, _vp, _sz, _vp],
    "nts_memcpy_d2h": [_vp, _vp, _sz, _int],
    "nts_memcpy_d2h_async": [_vp, _vp, _sz, _vp],
    "nts_memcpy_d2d_async": [_vp, _vp, _sz, _vp],
    "nts_memset_zero": [_vp, _sz, _vp],
    "nts_stream_create": [ctypes.POINTER(_vp)],
    "nts_stream_destroy": [_vp],
    "nts_stream_sync": [_vp],
    "nts_device_sync": [],
    "nts_mem_info": [ctypes.POINTER(_sz), ctypes.POINTER(_sz)],
    "nts_fingerprint_u32": [ctypes.POINTER(_u64), _vp, _u64, _vp, _u64, _vp],
    "nts_fingerprint_u32_async": [_vp, _vp, _u64, _vp, _u64, _vp],
    "nts_fingerprint_finish": [_u64, _u64, _u64],
    "nts_event_create": [ctypes.POINTER(_vp)],
    "nts_event_destroy": [_vp],
    "nts_event_record": [_vp, _vp],
    "nts_stream_wait_event": [_vp, _vp],
    "nts_event_elapsed_ms": [ctypes.POINTER(_f32), _vp, _vp],
    "nts_spmm_plan_set_events": [_vp, _vp, _vp],
    "nts_spmm_gather": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _int, _vp],
    "nts_spmm_gather_bounded": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _int, _u32, _vp],
    "nts_spmm_gather_static_scratch": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _int, _vp],
    "nts_spmm_plan_create": [ctypes.POINTER(_vp), _vp, _u32, _u32, _u32, _vp],
    "nts_spmm_plan_create_slabs": [ctypes.POINTER(_vp), _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, _vp],
    "nts_spmm_plan_schedule_host": [_vp, _vp, _u32, _u32, _u32, _u32, _vp, _u64, ctypes.POINTER(_u32),
                                    ctypes.POINTER(_u32), ctypes.POINTER(_u32)],
    "nts_spmm_plan_destroy": [_vp],
    "nts_spmm_plan_copy_schedule": [_vp, _vp, _u64, _vp, _u64],
    "nts_spmm_plan_info": [_vp, ctypes.POINTER(_u32), ctypes.POINTER(_u32), ctypes.POINTER(_u32)],
    "nts_spmm_plan_scratch_info": [_vp, _u32, ctypes.POINTER(_sz), ctypes.POINTER(_sz), ctypes.POINTER(_u64),
                                   ctypes.POINTER(_int)],
    "nts_spmm_plan_reserve": [_vp, _u32],
    "nts_spmm_gather_planned": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _int, _vp],
    "nts_scatter_src_to_edge": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp],
    "nts_scatter_dst_to_edge": [_vp, _vp, _vp, _u32, _u32, _vp],
    "nts_scatter_grad_to_edge": [_vp, _vp, _vp, _u32, _u32, _vp],
    "nts_gather_edge_to_dst": [_vp, _vp, _vp, _u32, _u32, _int, _vp],
    "nts_gather_edge_to_src": [_vp, _vp, _vp, _vp, _u32, _u32, _int, _vp],
    "nts_gather_edge_to_src_unsorted": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp],
    "nts_edge_softmax_fwd": [_vp, _vp, _vp, _u32, _u32, _vp],
    "nts_edge_softmax_bwd": [_vp, _vp, _vp, _vp, _u32, _u32, _vp],
    "nts_gat_attention_fwd": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _f32, _vp],
    "nts_gat_attention_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _f32, _vp],
    "nts_gat_attention_fwd_bounded": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _f32, _u32, _vp],
    "nts_gat_attention_bwd_bounded": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _f32, _u32, _vp],
    "nts_spmm_gather_heads": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _int, _vp],
    "nts_spmm_gather_heads_bounded": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _int, _u32, _vp],
    "nts_spmm_gather_heads_planned": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _int, _vp],
    "nts_sddmm_heads": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp],
    "nts_gather_rows_f32": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp],
    "nts_gather_rows_cached_f32": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp, _vp],
    "nts_gather_labels_i64": [_vp, _vp, _vp, _u32, _u32, _vp],
    "nts_message_rows_unpack": [_vp, _vp, _u32, _u32, _u32, _u32, _vp],
    "nts_message_rows_add": [_vp, _vp, _u32, _u32, _u32, _u32, _vp],
    "nts_sample_hop_work_bytes": [_u32],
    "nts_sample_hop_offsets": [_vp, _vp, _vp, _u32, ctypes.c_int32, _vp, _vp],
    "nts_sample_hop_neighbors": [_vp, _vp, _vp, _vp, _vp, _u32, ctypes.c_int32, ctypes.c_uint64, _vp],
    "nts_batch_builder_arena_bytes": [_u32, _u32, ctypes.POINTER(ctypes.c_int32), _u32, _u32, _int],
    "nts_batch_builder_create": [ctypes.POINTER(_vp), _vp, _vp, _u32, _u32, ctypes.POINTER(ctypes.c_int32), _u32, _u32,
                                 _int, _vp, _sz],
    "nts_batch_builder_sample": [_vp, _vp, _u32, _u64, _vp],
    "nts_batch_builder_layers": [_vp, _vp],
    "nts_batch_builder_use_graph": [_vp, ctypes.c_int],
    "nts_batch_builder_join": [_vp, _vp],
    "nts_batch_builder_destroy": [_vp],
    "nts_relabel_sources_work_bytes": [_u32],
    "nts_relabel_sources": [_vp, _vp, _vp, _vp, _u32, _u32, _vp, _vp],
    "nts_csr_from_csc_work_bytes": [_u32, _u32, _u32],
    "nts_csr_from_csc": [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp, _vp],
    "nts_gcn_edge_weights": [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp],
    "nts_chunk_from_edges_work_bytes": [_u32, _u32],
    "nts_chunk_from_edges": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp, _vp],
    "nts_edge_file_count": [_str, ctypes.POINTER(_u64)],
    "nts_edge_file_read": [_str, _vp, _u64, _u64, ctypes.POINTER(_u32)],
    "nts_read_feature_label_mask": [_str, _str, _str, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _int],
    "nts_feature_text_write": [_str, _vp, _vp, _u32, _u32, _int, _int],
    "nts_feature_csv_read": [_str, _vp, _u32, _u32, _int],
    "nts_int_list_text_read": [_str, _vp, _u64, ctypes.POINTER(_u64)],
    "nts_table_bin_write": [_str, _vp, _u64, _u64, _u32],
    "nts_table_bin_info": [_str, ctypes.POINTER(_u64), ctypes.POINTER(_u64), ctypes.POINTER(_u32)],
    "nts_table_bin_read": [_str, _vp, _u64, _u64],
}
_RESTYPES = {"nts_last_error": ctypes.c_char_p, "nts_fingerprint_finish": _u64, "nts_csr_from_csc_work_bytes": _sz,
             "nts_relabel_sources_work_bytes": _sz, "nts_sample_hop_work_bytes": _sz,
             "nts_chunk_from_edges_work_bytes": _sz, "nts_batch_builder_arena_bytes": _sz,
             "nts_trace_ranges_emitted": ctypes.c_long, "nts_scratch_alloc_count": ctypes.c_long}
# Entry points whose int result is a value, not a status.
_NO_STATUS = {"nts_last_error", "nts_abi_version", "nts_fingerprint_finish", "nts_scratch_alloc_count", "nts_trace_ranges_emitted", "nts_csr_from_csc_work_bytes", "nts_relabel_sources_work_bytes",
              "nts_sample_hop_work_bytes", "nts_chunk_from_edges_work_bytes", "nts_batch_builder_arena_bytes"}


class SampledLayerDesc(ctypes.Structure):
    """nts_sampled_layer_t of include/nts_hip.h."""
    _fields_ = [("v_size", _u32), ("e_size", _u32), ("src_size", _u32), ("max_in_degree", _u32),
                ("destination", _vp), ("source", _vp), ("column_offset", _vp), ("row_indices", _vp),
                ("row_offset", _vp), ("column_indices", _vp), ("csr_to_csc", _vp),
                ("edge_weight_forward", _vp), ("edge_weight_backward", _vp)]


class NtsError(RuntimeError):
    def __init__(self, name, code, text):
        super().__init__(f"{name} failed with status {code}: {text}")
        self.code = code


def build():
    """Compile lib/libntship.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", CSRC_DIR, "-j8", "-s"], check=True)


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: nothing else can compute these ops."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` (or __graft_entry__.build()); "
                "there is no fallback implementation"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, _int)
        _lib = handle
    return _lib


def ptr(x):
    if x is None:
        return 0
    if isinstance(x, int):
        return x
    return x.data_ptr()


def last_error():
    return lib().nts_last_error().decode()


def call(name, *args):
    """Calls an entry point and raises NtsError on a non-zero status."""
    if name not in SIGNATURES:
        raise KeyError(f"{name} has no entry in abi.SIGNATURES (arguments would be passed untyped)")
    fn = getattr(lib(), name)
    rc = fn(*args)
    if name not in _NO_STATUS and rc != NTS_OK:
        raise NtsError(name, rc, last_error())
    return rc


def status(name, *args):
    """Calls an entry point and returns its raw status (for tests of the error paths)."""
    return getattr(lib(), name)(*args)
