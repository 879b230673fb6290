"""``HistoryTrainer`` over a dataset directory: epochs of the ordinary and of the recorded loop, evaluation on the
validation and test splits with the feature cache only, the bookkeeping the reference's trainer keeps."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dataset(tmp_path, rng, N=6000, Fin=32, C=4):
    """62% of the nodes train, 18% validate, 20% test."""
    from hiscache import write_processed
    deg = 10
    indptr = np.arange(0, (N + 1) * deg, deg, dtype=np.int64)
    indices = rng.integers(0, N, size=N * deg).astype(np.int64)
    feats = rng.standard_normal((N, Fin)).astype(np.float32)
    labels = feats[:, :C].argmax(1).astype(np.int64)              # a node's own features decide its label
    perm = rng.permutation(N)
    write_processed(tmp_path, indptr, indices, feats, hot_ids=rng.permutation(N), labels=labels,
                    train_idx=perm[: N * 37 // 60], valid_idx=perm[N * 37 // 60: N * 4 // 5], test_idx=perm[N * 4 // 5:])
    return feats, labels


@pytest.mark.parametrize("recorded,placement,ring,read_ahead",
                         [(False, "host", False, False), (True, "host", False, False), (True, "hot", False, True),
                          (False, "device", False, False), (False, "hot", True, True), (True, "host", True, True),
                          (False, "host", False, True)])
def test_trainer_trains_and_evaluates(tmp_path, recorded, placement, ring, read_ahead):
    from hiscache import HistoryTrainer, make_config
    rng = np.random.default_rng(77)
    Fin, H, C, L = 32, 32, 4, 3
    dataset(tmp_path, rng, Fin=Fin, C=C)
    cfg = make_config(Fin, C, H, L, method="grad", rate=0.6, staleness_thres=5, device=DEV, path=str(tmp_path))
    torch.manual_seed(7)
    trainer = HistoryTrainer(cfg, fanout=[4, 3, 2], batch_size=200, lr=1e-2, num_epochs=3, eval_begin=1,
                             features_in_device_memory=placement == "device",
                             hot_rows=1500 if placement == "hot" else 0, cache_bytes=1500 * 32 * 4,
                             ring_rows=3000 if ring else 0, recorded=recorded, read_ahead=read_ahead)
    assert trainer.table.total_num_node == 6000 and set(trainer.splits) == {"train", "val", "test"}
    assert (trainer.uvm.hot_rows is not None) == (placement == "hot")
    trainer.train()
    assert trainer.glb_iter == 3 * 19                              # 3 700 training nodes in batches of 200
    assert len(trainer.val_metrics) == 2 and len(trainer.test_metrics) == 2 and len(trainer.epoch_seconds) == 3
    assert trainer.best_metric == max(trainer.val_metrics)
    assert trainer.val_metrics[-1] > 0.5 and trainer.test_metrics[-1] > 0.5    # four classes: chance is 0.25
    assert type(trainer.table).__name__ == ("RingHistoryCache" if ring else "HistoryCache")
    assert trainer.table.header > 0                                 # rows were admitted
    if recorded:
        if read_ahead:                                              # rows read straight into the recordings' arrays
            assert any(k[2] >= 0 and v[2] for k, v in trainer._step.shapes().items()), trainer._step.shapes()
        assert trainer._step.replays >= 30, trainer._step.shapes()  # (the nineteenth batch of an epoch is shorter)
    assert not trainer.model.training                                # left in evaluation mode, as the reference leaves it
    trainer.close()


def test_trainer_reads_its_settings_from_the_configuration(tmp_path):
    from hiscache import Config, HistoryTrainer, make_config
    rng = np.random.default_rng(78)
    dataset(tmp_path, rng, N=2000)
    cfg = make_config(32, 4, 32, 2, device=DEV, path=str(tmp_path))     # (two layers: hidden width = feature width)
    cfg["dl"]["sampler"] = Config({"train": {"batch_size": 128, "num_neighbors": [3, 2]}})
    cfg["train"]["train"] = Config({"num_epochs": 2, "eval_begin": 5})
    cfg["train"]["optimizer"] = Config({"lr": 0.003})
    trainer = HistoryTrainer(cfg, cache_bytes=400 * 32 * 4)
    assert trainer.batch_size == 128 and trainer.num_epochs == 2 and trainer.eval_begin == 5
    assert trainer.optimizer.param_groups[0]["lr"] == 0.003
    trainer.train()
    assert trainer.val_metrics == [] and len(trainer.epoch_seconds) == 2     # evaluation begins at epoch 5
    with pytest.raises(ValueError):          # a recording needs admission by gradient
        HistoryTrainer(make_config(32, 4, 32, 2, method="random", device=DEV, path=str(tmp_path)), fanout=[3, 2],
                       cache_bytes=400 * 32 * 4, recorded=True)
    with pytest.raises(ValueError):
        HistoryTrainer(make_config(32, 4, 32, 2, device=DEV, path=str(tmp_path)), fanout=[3], cache_bytes=400 * 32 * 4)


@pytest.mark.parametrize("recorded", [False, True])
def test_trainer_with_a_relational_model(tmp_path, recorded):
    """A model factory in place of ``get_model``: the relational model with node-type ranges of this dataset (three
    node types, five relations from the type pairs); the sampler then emits the view's edge slots too."""
    from hiscache import HistoryRGCN, HistoryTrainer, make_config
    rng = np.random.default_rng(79)
    N, Fin, H, C, L, K = 6000, 32, 32, 4, 2, 5
    dataset(tmp_path, rng, N=N, Fin=Fin, C=C)
    cfg = make_config(Fin, C, H, L, method="grad", rate=0.6, staleness_thres=5, device=DEV, path=str(tmp_path),
                      model_type="rgcn", num_rel=K, name="rmag240m")

    def factory(config, table):
        return HistoryRGCN(Fin, H, C, L, 0.0, "CSR_Layer", config, table, num_rel=K, dataset_name="rmag240m",
                           type_bounds=[N // 2, N - 500], pair_to_rel=[[0, 1, 0], [2, 0, 3], [0, 4, 0]])

    torch.manual_seed(8)
    trainer = HistoryTrainer(cfg, fanout=[5, 4], batch_size=200, lr=1e-2, num_epochs=3, eval_begin=2,
                             cache_bytes=1500 * 32 * 4, recorded=recorded, model_factory=factory)
    assert trainer.sampler.view_edges
    trainer.train()
    assert len(trainer.val_metrics) == 1 and trainer.test_metrics == []      # (no test epoch for the mag datasets)
    # (labels decided by a node's own features are out of reach of a model without a self term: only the run counts)
    assert 0.0 <= trainer.val_metrics[0] <= 1.0 and trainer.table.header > 0
    assert all(torch.isfinite(p).all() for p in trainer.model.parameters())
    if recorded:
        assert trainer._step.replays >= 30, trainer._step.shapes()


def test_trainer_without_the_embedding_cache(tmp_path):
    """``feat_mode = "uvm"``: features through the store, no embedding is cached or admitted
    (/root/reference/hiscache/history_cache.py:290-304)."""
    from hiscache import HistoryTrainer, make_config
    rng = np.random.default_rng(80)
    dataset(tmp_path, rng)
    cfg = make_config(32, 4, 32, 3, device=DEV, path=str(tmp_path), feat_mode="uvm")
    torch.manual_seed(3)
    trainer = HistoryTrainer(cfg, fanout=[4, 3, 2], batch_size=200, lr=1e-2, num_epochs=3, eval_begin=2,
                             cache_bytes=400 * 32 * 4)
    trainer.train()
    assert trainer.table.header == 0 and len(trainer.val_metrics) == 1 and trainer.val_metrics[0] > 0.4


@pytest.mark.parametrize("method", ["random", "staleness"])
def test_trainer_with_the_other_admission_policies(tmp_path, method):
    """``history.method`` other than "grad": scores are drawn at random, no gradient of the embeddings is kept
    (/root/reference/hiscache/history_cache.py:205-215)."""
    from hiscache import HistoryTrainer, make_config
    rng = np.random.default_rng(81)
    dataset(tmp_path, rng)
    cfg = make_config(32, 4, 32, 3, method=method, rate=0.5, staleness_thres=7, device=DEV, path=str(tmp_path))
    torch.manual_seed(4)
    trainer = HistoryTrainer(cfg, fanout=[4, 3, 2], batch_size=200, lr=1e-2, num_epochs=3, eval_begin=2,
                             cache_bytes=1500 * 32 * 4)
    trainer.train()
    assert trainer.table.header > 0 and trainer.val_metrics[0] > 0.4


@pytest.mark.parametrize("recorded", [False, True])
def test_trainer_keeps_half_precision_features_in_half_precision(tmp_path, recorded):
    from hiscache import HistoryTrainer, ProcessedDataset, make_config, write_processed
    rng = np.random.default_rng(82)
    N, Fin, C = 6000, 32, 4
    indptr = np.arange(0, (N + 1) * 10, 10, dtype=np.int64)
    indices = rng.integers(0, N, size=N * 10).astype(np.int64)
    feats = rng.standard_normal((N, Fin)).astype(np.float16)
    perm = rng.permutation(N)
    write_processed(tmp_path, indptr, indices, feats, hot_ids=rng.permutation(N),
                    labels=feats[:, :C].argmax(1).astype(np.int64), train_idx=perm[:3600], valid_idx=perm[3600:4800])
    cfg = make_config(Fin, C, 32, 3, method="grad", rate=0.5, staleness_thres=7, device=DEV, path=str(tmp_path))
    torch.manual_seed(5)
    trainer = HistoryTrainer(cfg, dataset=ProcessedDataset(tmp_path, Fin, feature_dtype=np.float16), fanout=[4, 3, 2],
                             batch_size=200, lr=1e-2, num_epochs=3, eval_begin=2, cache_bytes=1500 * 32 * 4,
                             hot_rows=1000, read_ahead=True, recorded=recorded)
    assert trainer.uvm.buffer.dtype == torch.float16 and trainer.uvm.out_dtype == torch.float16
    assert trainer.uvm.hot_rows.dtype == torch.float16
    trainer.train()
    assert trainer.val_metrics[0] > 0.5 and trainer.table.header > 0
    trainer.close()


def test_profiled_epoch_reports_the_phases(tmp_path):
    """``dl.performance.prof``: ``train`` runs the profiled epoch, which sums the time of every phase as the
    reference's does (load, forward, loss, backward, step, update, sample) and trains like the ordinary one."""
    from hiscache import Config, HistoryTrainer, make_config
    rng = np.random.default_rng(83)
    dataset(tmp_path, rng)
    cfg = make_config(32, 4, 32, 3, method="grad", rate=0.5, staleness_thres=7, device=DEV, path=str(tmp_path))
    cfg["dl"]["performance"] = Config({"prof": True})
    torch.manual_seed(6)
    trainer = HistoryTrainer(cfg, fanout=[4, 3, 2], batch_size=200, lr=1e-2, num_epochs=2, eval_begin=1,
                             cache_bytes=1500 * 32 * 4)
    assert trainer.prof
    trainer.train()
    assert set(trainer.times) == {"load", "forward", "loss", "backward", "step", "update", "sample"}
    assert all(v >= 0.0 for v in trainer.times.values()) and trainer.times["forward"] > 0 and trainer.times["backward"] > 0
    assert sum(trainer.times.values()) < 2.0 * trainer.epoch_seconds[-1] + 0.1
    assert trainer.glb_iter == 2 * 19 and trainer.val_metrics[0] > 0.5 and trainer.table.header > 0


@pytest.mark.parametrize("ring,recorded", [(False, False), (True, False), (False, True)])
def test_checkpoint_and_resume_continue_the_same_run(tmp_path, ring, recorded):
    """Two epochs in one go against one epoch, ``state_dict`` through ``torch.save`` / ``torch.load``, a fresh
    trainer, ``load_state_dict`` and the second epoch: the same parameters, cache contents and counters, bit for
    bit (the sampler's batch keys and the shuffling generator continue where they stopped)."""
    from hiscache import HistoryTrainer, make_config
    rng = np.random.default_rng(84)
    dataset(tmp_path, rng)
    cfg = make_config(32, 4, 32, 3, method="grad", rate=0.5, staleness_thres=7, device=DEV, path=str(tmp_path))

    def build():
        torch.manual_seed(9)
        return HistoryTrainer(cfg, fanout=[4, 3, 2], batch_size=200, lr=1e-2, num_epochs=2, eval_begin=9,
                              cache_bytes=1500 * 32 * 4, ring_rows=3000 if ring else 0, recorded=recorded, seed=3)

    whole = build()
    whole.cxg_train_epoch()
    whole.cxg_train_epoch()
    first = build()
    first.cxg_train_epoch()
    path = str(tmp_path / "checkpoint.pt")
    torch.save(first.state_dict(), path)
    resumed = build()
    resumed.load_state_dict(torch.load(path, weights_only=True))
    assert resumed.glb_iter == first.glb_iter == 19
    resumed.cxg_train_epoch()
    assert resumed.glb_iter == whole.glb_iter == 38
    for p, q in zip(resumed.model.parameters(), whole.model.parameters()):
        assert torch.equal(p, q)
    a, b = resumed.table.state_dict(), whole.table.state_dict()
    assert set(a) == set(b)
    for k in a:
        assert (torch.equal(a[k], b[k]) if isinstance(a[k], torch.Tensor) else a[k] == b[k]), k
    other = HistoryTrainer(cfg, fanout=[4, 3, 2], batch_size=200, cache_bytes=700 * 32 * 4, ring_rows=1000 if ring else 0)
    with pytest.raises(ValueError):
        other.table.load_state_dict(first.table.state_dict())      # a cache of another size


@pytest.mark.parametrize("extra", [[], ["trainer.recorded=true", "trainer.read_ahead=true", "trainer.hot_rows=2000"]])
def test_example_main_trains_from_its_configuration(tmp_path, extra):
    """The example's entry (the role of /root/reference/example/main.py): YAML configuration, overrides, a dataset
    written on request, ``HistoryTrainer(config).train()``."""
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location(
        "hiscache_example_main", os.path.join(here, "..", "history-cache_amd", "example", "main.py"))
    ex = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ex)
    trainer = ex.main(["--synthetic", "8000", f"dl.dataset.path={tmp_path}", "dl.dataset.feature_dim=32",
                       "dl.dataset.num_classes=4", "train.model.hidden_dim=32", "dl.sampler.train.batch_size=400",
                       "dl.sampler.train.num_neighbors=[4,3,2]", "train.optimizer.lr=0.01", "history.rate=0.6",
                       "history.staleness_thres=5", "trainer.cache_megabytes=0.25", "train.train.num_epochs=3"] + extra)
    assert trainer.glb_iter == 3 * 12                              # 4 800 training nodes in batches of 400
    assert len(trainer.val_metrics) == 3 and trainer.val_metrics[-1] > 0.5 and trainer.test_metrics[-1] > 0.5
    assert trainer.recorded == bool(extra) and (trainer.uvm.hot_rows is not None) == bool(extra)
    assert os.path.exists(os.path.join(tmp_path, "processed", "sorted_indices.dat"))


def test_just_load_hit_rates_and_batch_file(tmp_path):
    """``cxg_just_load`` (/root/reference/hiscache/history_trainer.py:144-174) against a dictionary model run over the
    same batches (a second trainer with the same seeds draws them again); ``batch_to_file`` round trip."""
    from hiscache import HistoryTrainer, make_config
    rng = np.random.default_rng(83)
    dataset(tmp_path, rng, N=3000)
    cfg = make_config(32, 4, 32, 2, device=DEV, path=str(tmp_path))

    def build():
        return HistoryTrainer(cfg, fanout=[4, 3], batch_size=150, cache_bytes=400 * 32 * 4, seed=3)

    def score(n):                                         # a fixed pseudo-random order of the positions
        return ((torch.arange(n, device=DEV) * 7919) % 1009).to(torch.float32)
    a, b = build(), build()
    got = a.cxg_just_load(num_epochs=2, rate=0.8, staleness=5, score_fn=score)
    count, window, want = {}, [], []
    for _ in range(2):
        for batch in b._batches(b.splits["train"], shuffle=True):
            nodes = batch.sub_to_full[: int(batch.num_node_in_layer[1])].tolist()
            held = [count.get(v, 0) > 0 for v in nodes]
            want.append((sum(held) / len(nodes), sum(1 for c in count.values() if c > 0)))
            sc = score(len(nodes))
            thres = float(torch.quantile(sc, 0.8))
            new = [v for v, s, h in zip(nodes, sc.tolist(), held) if s < thres and not h]
            window.append(new)
            if len(window) > 5:
                for v in window.pop(0):
                    count[v] -= 1
            for v in new:
                count[v] = count.get(v, 0) + 1
    assert len(got) == 2 * 13 and a.glb_iter == 26         # 1 850 training nodes in batches of 150
    assert [g[1] for g in got] == [w[1] for w in want]
    np.testing.assert_allclose([g[0] for g in got], [w[0] for w in want], rtol=1e-6)
    assert got[0] == (0.0, 0) and max(g[0] for g in got) > 0.05
    # with the default scores it runs from the trainer's generator
    assert len(a.cxg_just_load(num_epochs=1)) == 13
    batch = a.sampler.sample(a.splits["train"][:100].contiguous())
    HistoryTrainer.batch_to_file(batch, tmp_path / "batch.pt")
    back = torch.load(tmp_path / "batch.pt", weights_only=True)
    assert torch.equal(back["ptr"], batch.ptr.cpu()) and torch.equal(back["idx"], batch.idx.cpu())
    assert back["num_node_in_layer"].tolist() == batch.num_node_in_layer.tolist()
    a.close(), b.close()
