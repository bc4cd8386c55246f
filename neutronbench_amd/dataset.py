"""Dataset files: mirror of GNNDatum's readers (core/ntsDataloador.hpp:209-471) and of the binary
edge list Graph::load_directed consumes (core/graph.hpp:1050-1061), over the C ABI.

Feature tables are read straight into page-locked host memory mapped into the device address space
(the reference's cudaMallocPinned, core/ntsDataloador.hpp:74-75), so the zero-copy feature gather
can use them without another copy.  Labels are int64, masks int32 (0 train, 1 val, 2 test, 3 other).
"""
import ctypes
import os

import numpy as np

from .abi import call


def _np_ptr(a):
    return a.ctypes.data if a is not None else 0


def _path(p):
    return os.fsencode(p)


class PinnedArray:
    """A numpy view of page-locked, device-mapped host memory owned by the library."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        host = ctypes.c_void_p()
        call("nts_malloc_pinned_mapped", ctypes.byref(host), max(nbytes, 1))
        self.host_ptr = host.value
        buf = (ctypes.c_ubyte * max(nbytes, 1)).from_address(self.host_ptr)
        self.array = np.frombuffer(buf, dtype=self.dtype, count=int(np.prod(self.shape))).reshape(self.shape)
        self.array[...] = 0
        dev = ctypes.c_void_p()
        call("nts_host_get_device_ptr", ctypes.byref(dev), self.host_ptr)
        self.dev_ptr = dev.value

    def close(self):
        if self.host_ptr:
            self.array = None
            call("nts_free_pinned", self.host_ptr)
            self.host_ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def edge_file_count(path):
    n = ctypes.c_uint64()
    call("nts_edge_file_count", _path(path), ctypes.byref(n))
    return n.value


def read_edge_file(path, vertices=None, out=None):
    """The .edge file's records as a uint32 array [E, 2] (columns src, dst).  `out` may be the
    array of a PinnedArray; `vertices`, when given, is checked against the largest id."""
    E = edge_file_count(path)
    pairs = out if out is not None else np.empty((E, 2), dtype=np.uint32)
    assert pairs.dtype == np.uint32 and pairs.size == 2 * E and pairs.flags.c_contiguous
    max_id = ctypes.c_uint32()
    call("nts_edge_file_read", _path(path), _np_ptr(pairs), 0, E, ctypes.byref(max_id))
    if vertices is not None and E and max_id.value >= vertices:
        raise ValueError(f"{path}: vertex id {max_id.value} but only {vertices} vertices")
    return pairs


def write_edge_file(path, pairs):
    np.ascontiguousarray(pairs, dtype=np.uint32).tofile(path)


def write_feature_file(path, features, ids=None, decimals=4, threads=0):
    """Text feature file as data/generate_nts_dataset.py writes it: one record per line,
    "id f0 f1 ... fF-1", values printed with `decimals` digits after the point (so the file holds the
    rounded values, which is what a reader then sees)."""
    features = np.ascontiguousarray(features, dtype=np.float32)
    V, F = features.shape
    ids32 = None if ids is None else np.ascontiguousarray(ids, dtype=np.uint32)
    call("nts_feature_text_write", _path(path), _np_ptr(features), _np_ptr(ids32) if ids32 is not None else 0, V, F,
         decimals, threads)


def write_label_file(path, labels, ids=None):
    """"id label" per line (single-label form)."""
    labels = np.asarray(labels).astype(np.int64)
    ids = np.arange(labels.size) if ids is None else np.asarray(ids)
    np.savetxt(path, np.stack([ids, labels], 1), fmt="%d")


MASK_WORDS = ("train", "val", "test")


def write_mask_file(path, mask, ids=None):
    """"id word" per line; mask values 0 / 1 / 2 are written as train / val / test, anything else
    as "unknown" (which the readers store as 3)."""
    mask = np.asarray(mask)
    ids = np.arange(mask.size) if ids is None else np.asarray(ids)
    with open(path, "w") as f:
        f.write("".join(f"{i} {MASK_WORDS[m] if 0 <= m < 3 else 'unknown'}\n" for i, m in zip(ids.tolist(), mask.tolist())))


class GNNDatum:
    """local_feature [V, F] float32, local_label / global_label int64, local_mask / global_mask int32
    of one partition that owns every vertex (core/ntsDataloador.hpp:36-88)."""

    def __init__(self, vertices, feature_size, classes=1, pinned=True):
        self.V, self.F, self.classes = int(vertices), int(feature_size), int(classes)
        width = self.classes if self.classes > 1 else 1
        self._pinned = PinnedArray((self.V, self.F), np.float32) if pinned else None
        self.local_feature = self._pinned.array if pinned else np.zeros((self.V, self.F), dtype=np.float32)
        self.local_label = np.zeros(self.V * width, dtype=np.int64)
        self.global_label = np.zeros(self.V * width, dtype=np.int64)
        self.local_mask = np.zeros(self.V, dtype=np.int32)
        self.global_mask = np.zeros(self.V, dtype=np.int32)

    @property
    def dev_local_feature(self):
        """Device-side address of the pinned feature table (getDevicePointer)."""
        if self._pinned is None:
            raise RuntimeError("feature table is not in mapped host memory")
        return self._pinned.dev_ptr

    def readFeature_Label_Mask(self, inputF, inputL, inputM, threads=0):
        """core/ntsDataloador.hpp:264-395."""
        call("nts_read_feature_label_mask", _path(inputF), _path(inputL), _path(inputM), self.V, self.F, self.classes,
             _np_ptr(self.local_feature), _np_ptr(self.local_label), _np_ptr(self.local_mask),
             _np_ptr(self.global_label), _np_ptr(self.global_mask), threads)

    def readFeature_Label_Mask_OGB(self, inputF, inputL, inputM, threads=0):
        """core/ntsDataloador.hpp:397-471: comma-separated features, one label per line, and the
        split id lists train.csv / valid.csv / test.csv under the directory inputM."""
        call("nts_feature_csv_read", _path(inputF), _np_ptr(self.local_feature), self.V, self.F, threads)
        n = ctypes.c_uint64()
        call("nts_int_list_text_read", _path(inputL), _np_ptr(self.local_label), self.V, ctypes.byref(n))
        for code, name in enumerate(("train.csv", "valid.csv", "test.csv")):
            p = os.path.join(inputM, name)
            call("nts_int_list_text_read", _path(p), 0, 0, ctypes.byref(n))
            ids = np.empty(max(n.value, 1), dtype=np.int64)
            call("nts_int_list_text_read", _path(p), _np_ptr(ids), n.value, ctypes.byref(n))
            ids = ids[: n.value]
            self.local_mask[ids[(ids >= 0) & (ids < self.V)]] = code

    def read_feature_table(self, path):
        """Binary table written by write_feature_table: no parsing, one read into the pinned table."""
        rows, cols, eb = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint32()
        call("nts_table_bin_info", _path(path), ctypes.byref(rows), ctypes.byref(cols), ctypes.byref(eb))
        if (rows.value, cols.value, eb.value) != (self.V, self.F, 4):
            raise ValueError(f"{path}: table is {rows.value} x {cols.value} x {eb.value} B, expected {self.V} x {self.F} x 4 B")
        call("nts_table_bin_read", _path(path), _np_ptr(self.local_feature), 0, self.V)

    def write_feature_table(self, path):
        call("nts_table_bin_write", _path(path), _np_ptr(self.local_feature), self.V, self.F, 4)

    def close(self):
        if self._pinned is not None:
            self.local_feature = None
            self._pinned.close()
            self._pinned = None
