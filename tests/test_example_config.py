"""The example's configuration loading: YAML tree, hydra-style overrides, the trainer's option group."""
import importlib.util
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXAMPLE = os.path.join(HERE, "..", "history-cache_amd", "example")


def load_example():
    spec = importlib.util.spec_from_file_location("hiscache_example_main", os.path.join(EXAMPLE, "main.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_the_shipped_configuration_holds_every_key_that_is_read():
    ex = load_example()
    cfg = ex.load_config(os.path.join(EXAMPLE, "config.yaml"))
    # the keys the reference reads: history_cache.py:13-36, history_table.py:12-30, history_trainer.py:17-45
    assert cfg.dl.dataset.feature_dim == 128 and cfg.dl.dataset.num_classes == 16 and cfg.dl.num_device == 1
    assert cfg.dl.loading.feat_mode == "history_uvm" and cfg.dl.type == "cxg" and cfg.train.type == "cxg"
    assert cfg.train.model.type == "sage" and cfg.train.model.num_layers == len(cfg.dl.sampler.train.num_neighbors)
    for key in ("method", "rate", "staleness_thres", "limit", "start_history", "distributed_store",
                "store_last_layer", "buffer_size", "graph_struct_norm"):
        assert key in cfg.history, key
    opts = ex.trainer_options(cfg)
    assert opts == dict(recorded=False, read_ahead=False, features_in_device_memory=False, hot_rows=0, ring_rows=0,
                        cache_bytes=None, seed=0)


def test_overrides(tmp_path):
    ex = load_example()
    cfg = ex.load_config(os.path.join(EXAMPLE, "config.yaml"),
                         ["history.rate=0.75", "trainer.recorded=true", "dl.sampler.train.num_neighbors=[4,3]",
                          "train.model.num_layers=2", "dl.dataset.path=/data/x", "trainer.cache_megabytes=1.5",
                          "extra.group.key=7"])
    assert cfg.history.rate == 0.75 and cfg.dl.sampler.train.num_neighbors == [4, 3]
    assert cfg.train.model.num_layers == 2 and cfg.dl.dataset.path == "/data/x" and cfg.extra.group.key == 7
    opts = ex.trainer_options(cfg)
    assert opts["recorded"] is True and opts["cache_bytes"] == 3 * 2 ** 19
    with pytest.raises(ValueError):
        ex.load_config(os.path.join(EXAMPLE, "config.yaml"), ["history.rate"])
    with pytest.raises(ValueError):
        ex.load_config(os.path.join(EXAMPLE, "config.yaml"), ["history.rate.deeper=1"])
    empty = tmp_path / "empty.yaml"
    empty.write_text("")
    assert ex.trainer_options(ex.load_config(str(empty)))["hot_rows"] == 0


def test_more_than_one_device_is_refused(tmp_path):
    ex = load_example()
    with pytest.raises(SystemExit):
        ex.main(["dl.num_device=2", f"dl.dataset.path={tmp_path}"])
