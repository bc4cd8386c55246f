"""The C-ABI library loads without a GPU and exports every entry point that include/nts_hip.h
declares (no compute calls here)."""
import ctypes
import os
import re

from neutronbench_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "nts_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nts_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_binds():
    assert _declared() == sorted(abi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(abi.LIB_PATH)
    missing = [name for name in _declared() if not hasattr(handle, name)]
    assert not missing, f"libntship.so lacks {missing}"


def test_version_and_host_side_argument_checks():
    assert abi.call("nts_abi_version") == 1
    # argument validation happens before any device work, so it can run without a GPU
    assert abi.status("nts_spmm_gather", 0, 0, 0, 0, 0, 0, 4, 0, 0, 0, 0) == abi.NTS_ERR_INVALID
    assert "F is 0" in abi.last_error()
    assert abi.status("nts_gather_labels_i64", 0, 0, 0, 4, 0, 0) == abi.NTS_ERR_INVALID
    assert abi.status("nts_edge_softmax_fwd", 0, 0, 0, 4, 0, 0) == abi.NTS_ERR_INVALID
    assert abi.status("nts_free_device", 0) == abi.NTS_OK  # free(NULL) is tolerated
    assert abi.status("nts_spmm_plan_destroy", 0) == abi.NTS_OK
    assert abi.status("nts_malloc_device", None, 16) == abi.NTS_ERR_INVALID
