"""Rows that arrive as message records {uint32 vertex id, F floats} (the exchange format of the
reference's full-graph GPU operators, cuda/ntsCUDATransferKernel.cuh:43-93): unpacking is a copy,
bit-exact; adding is a sum per row -- exact for distinct rows (one addition per element), and in
record order when a buffer names a row more than once."""
import numpy as np
import pytest
import torch

from gpu_util import dev, stream
from neutronbench_amd import abi
from neutronbench_amd.abi import call, ptr
from neutronbench_amd.batch import MappedHostTable

pytestmark = pytest.mark.gpu


def records(ids, values):
    rec = np.empty((ids.size, values.shape[1] + 1), dtype=np.float32)
    rec[:, 0] = ids.astype(np.uint32).view(np.float32)
    rec[:, 1:] = values
    return rec


@pytest.mark.parametrize("F", [1, 7, 64, 128, 602])
def test_unpack_and_add_distinct_rows(device, F):
    rng = np.random.default_rng(F)
    lo, hi, n = 1000, 6000, 3000
    ids = rng.permutation(np.arange(lo - 200, hi + 200))[:n]  # some ids fall outside [lo, hi): skipped
    vals = rng.standard_normal((n, F)).astype(np.float32)
    rec = records(ids, vals)
    inside = (ids >= lo) & (ids < hi)
    init = rng.standard_normal((hi - lo, F)).astype(np.float32)
    want_unpack = init.copy()
    want_unpack[ids[inside] - lo] = vals[inside]
    want_add = init.copy()
    want_add[ids[inside] - lo] += vals[inside]
    for source in ("device", "mapped host"):
        if source == "device":
            drec = dev(rec, device)
            rec_ptr = ptr(drec)
        else:
            table = MappedHostTable(torch.from_numpy(rec))
            rec_ptr = table.dev_ptr
        rows = dev(init, device)
        call("nts_message_rows_unpack", ptr(rows), rec_ptr, n, F, lo, hi, stream())
        torch.cuda.synchronize()
        assert rows.cpu().numpy().tobytes() == want_unpack.tobytes(), source
        rows = dev(init, device)
        call("nts_message_rows_add", ptr(rows), rec_ptr, n, F, lo, hi, stream())
        torch.cuda.synchronize()
        assert rows.cpu().numpy().tobytes() == want_add.tobytes(), source
        if source != "device":
            table.close()


def test_add_with_repeated_rows_follows_record_order(device):
    rng = np.random.default_rng(5)
    F, rows_n, n = 33, 50, 4000
    ids = rng.integers(0, rows_n, n)
    vals = rng.standard_normal((n, F)).astype(np.float32)
    want = np.zeros((rows_n, F), dtype=np.float32)
    for k in range(n):  # the running fp32 sum in record order
        want[ids[k]] += vals[k]
    drec = dev(records(ids, vals), device)
    outs = []
    for _ in range(2):
        rows = torch.zeros(rows_n, F, device=device)
        call("nts_message_rows_add", ptr(rows), ptr(drec), n, F, 0, rows_n, stream())
        torch.cuda.synchronize()
        outs.append(rows.cpu().numpy())
    assert outs[0].tobytes() == want.tobytes() and outs[1].tobytes() == want.tobytes()


def test_empty_and_invalid(device):
    s = stream()
    rows = torch.ones(4, 3, device=device)
    call("nts_message_rows_unpack", ptr(rows), 0, 0, 3, 0, 4, s)
    call("nts_message_rows_add", ptr(rows), 0, 0, 3, 0, 4, s)
    assert abi.status("nts_message_rows_add", ptr(rows), 0, 5, 3, 0, 4, s) == abi.NTS_ERR_INVALID
    assert abi.status("nts_message_rows_unpack", ptr(rows), ptr(rows), 5, 0, 0, 4, s) == abi.NTS_ERR_INVALID
    torch.cuda.synchronize()
    assert bool((rows == 1).all())
