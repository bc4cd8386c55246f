"""Host logic of the epoch runners that needs no GPU."""
from neutronbench_amd import epoch


def test_graph_mode_picked_by_batches_in_flight_and_feature_cache():
    """nts_batch_builder_use_graph value of the epoch loops: an explicit value is passed through; True
    picks the one recorded chain with several batches in flight, and with one batch in flight the
    second graph beside the gather."""
    assert epoch.graph_mode(True, 1, 0.2) == 3
    assert epoch.graph_mode(True, 1, 0.0) == 3
    assert epoch.graph_mode(True, 1) == 3
    for p in (2, 3, 4, 6):
        assert epoch.graph_mode(True, p, 0.2) == 1
        assert epoch.graph_mode(True, p, 0.0) == 1
    for explicit in (0, 1, 2, 3):
        assert epoch.graph_mode(explicit, 1, 0.2) == explicit
        assert epoch.graph_mode(explicit, 4, 0.0) == explicit
    assert epoch.graph_mode(False, 1, 0.2) == 0


def test_every_configuration_names_what_the_native_driver_needs():
    for name, cfg in epoch.CONFIGS.items():
        for key in ("V", "E", "F", "hidden", "classes", "fanout", "batch", "train", "seed", "cache"):
            assert key in cfg, (name, key)
        assert cfg["hidden"] % max(cfg.get("heads", 0), 1) == 0
        assert all(f != 0 for f in cfg["fanout"]) and 1 <= len(cfg["fanout"]) <= 8
