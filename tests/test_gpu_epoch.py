"""The epoch harness gives the same batches whatever the number of batches in flight: the pipelined
modes (sampling, gather and aggregation of consecutive batches on streams of their own, ordered by
events) must reproduce the serial mode's sampled edges, gathered rows, cache hits and a checksum of
every batch's aggregation output and input gradient, bit for bit."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("config,scale", [("arxiv", 0.25), ("products", 0.02), ("gat", 0.02)])
def test_pipelined_epochs_match_the_serial_one(config, scale):
    from neutronbench_amd import epoch

    runs = {p: epoch.run(config, scale=scale, max_batches=7, warmup_batches=1, pipeline=p, quiet=True, checksum=True)
            for p in (1, 2, 3, 5)}
    serial = runs[1]
    assert serial["sampled_edges"] > 0 and serial["gathered_rows"] > 0 and serial["checksum"] != 0.0
    for p, r in runs.items():
        assert r["pipeline"] == p
        for key in ("batches", "sampled_edges", "gathered_rows", "cache_hit_rate", "checksum"):
            assert r[key] == serial[key], (p, key, r[key], serial[key])


def test_pipelined_epoch_without_warm_up_batches():
    from neutronbench_amd import epoch

    a = epoch.run("arxiv", scale=0.25, max_batches=3, warmup_batches=0, pipeline=1, quiet=True, checksum=True)
    for p in (2, 4):
        b = epoch.run("arxiv", scale=0.25, max_batches=3, warmup_batches=0, pipeline=p, quiet=True, checksum=True)
        assert (b["sampled_edges"], b["checksum"]) == (a["sampled_edges"], a["checksum"])


def test_two_batches_in_flight_without_stage_waits():
    """With two batches in flight and no host-side wait between the stages, the sampling of batch k+2
    re-uses the arena batch k was built in while batch k may still be aggregated: the sampling stream
    waits for an event recorded after that aggregation.  Same results as the serial epoch."""
    from neutronbench_amd import epoch

    a = epoch.run("products", scale=0.05, max_batches=8, warmup_batches=0, pipeline=1, quiet=True, checksum=True)
    b = epoch.run("products", scale=0.05, max_batches=8, warmup_batches=0, pipeline=2, stage_sync=False, quiet=True,
                  checksum=True)
    for key in ("sampled_edges", "gathered_rows", "cache_hit_rate", "checksum"):
        assert a[key] == b[key], (key, a[key], b[key])


def test_hop_by_hop_sampler_builds_the_same_batches():
    from neutronbench_amd import epoch

    a = epoch.run("arxiv", scale=0.25, max_batches=5, warmup_batches=0, sampler="builder", quiet=True, checksum=True)
    b = epoch.run("arxiv", scale=0.25, max_batches=5, warmup_batches=0, sampler="library", quiet=True, checksum=True)
    for key in ("sampled_edges", "gathered_rows", "checksum"):
        assert a[key] == b[key], (key, a[key], b[key])


def test_stream_wrapper_can_leave_batch_assembly_unsynchronised():
    import torch

    from neutronbench_amd.stream import CudaStream

    dev = torch.device("cuda:0")
    table = torch.arange(64 * 8, dtype=torch.float32, device=dev).view(64, 8)
    ids = torch.tensor([5, 0, 63, 5], dtype=torch.int32, device=dev)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream())
    out = torch.zeros(4, 8, device=dev)
    with torch.cuda.stream(side):
        cs = CudaStream(side.cuda_stream, synchronize=False)
        cs.zero_copy_feature_move_gpu(out, table, ids, 8, 4)
        done = torch.cuda.Event()
        done.record(side)
    torch.cuda.current_stream().wait_event(done)
    assert torch.equal(out, table[ids.long()])
    assert CudaStream(side.cuda_stream).synchronize is True


@pytest.mark.parametrize("config,scale", [("arxiv", 0.25), ("products", 0.02), ("gat", 0.02)])
def test_native_epoch_driver(config, scale):
    """The epoch driven from C++ (lib/nts_epoch, neutronbench_amd/host/epoch_driver.cpp): same graph,
    train ids and seeds as the Python loop, so it samples the same edges, gathers the same rows and
    hits the cache as often; its checksum of every aggregation output (a device-side hash per layer
    and direction) is the same for every number of batches in flight, without graph replay and with each of its three
    shapes (one chain; transpositions on a side branch; transpositions as a second graph on the builder's own
    stream, joined before the aggregation)."""
    from neutronbench_amd import epoch

    py = epoch.run(config, scale=scale, max_batches=7, warmup_batches=1, quiet=True)
    runs = [epoch.run_native(config, scale=scale, max_batches=7, warmup_batches=1, pipeline=p, graph=g, quiet=True,
                             verify=True)
            for p, g in ((1, True), (1, False), (1, 1), (1, 2), (1, 3), (2, True), (2, 3), (3, True), (5, True), (4, 3))]
    for r in runs:
        assert r["batches"] == py["batches"]
        assert r["sampled_edges"] == py["sampled_edges"] and r["gathered_rows"] == py["gathered_rows"]
        assert r["checksum"] == runs[0]["checksum"]
    if py["cache_hit_rate"] is not None:
        assert abs(runs[0]["cache_hit_rate"] - py["cache_hit_rate"]) < 1e-4


@pytest.mark.parametrize("config,scale", [("arxiv", 0.25), ("products", 0.02), ("gat", 0.02)])
def test_native_epoch_batch_against_the_oracle(config, scale, tmp_path):
    """Every array of one batch of the native epoch -- sampled layers, CSR, weights, gathered features
    and labels, each aggregation's (or GAT operator's) input and output, as written by --dump-dir after
    the timed epoch -- against the CPU oracle: structure and gathers bit for bit, sums within 1e-4."""
    from neutronbench_amd import epoch
    from oracle import epoch_check

    data, dump = tmp_path / "data", tmp_path / "dump"
    data.mkdir()
    dump.mkdir()
    host = epoch.write_native_inputs(config, str(data), scale, keep_host=True)
    cfg = epoch.CONFIGS[config]
    n_batches = min(4, -(-host["n_train"] // cfg["batch"]))
    out = epoch.run_native_on(str(data), config, host["V"], max_batches=4, warmup_batches=1, stage_sync=True,
                              dump_dir=str(dump), dump_batch=n_batches - 1)
    assert out["batches"] == n_batches
    assert set(out["stage_s"]) == {"sample", "gather", "aggregate_fwd", "aggregate_bwd"}
    res = epoch_check.check_dump(str(dump), host["co"], host["ri"], host["feat"], host["labels"], cfg["fanout"],
                                 cfg["cache"])
    assert res["ok"], res
    assert res["sampled_edges"] > 0 and res["checked_rows"] > 0 and res["max_rel_err"] <= 1e-4
    if not cfg.get("heads"):
        assert res["bit_exact_rows"] > 0
