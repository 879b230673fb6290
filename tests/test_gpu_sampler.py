"""hc_sample_layers through the C ABI against the sequential CPU statement: ptr, idx, sub_to_full
and the layer sizes bit-exact."""
import numpy as np
import pytest
import torch

from test_oracle_sampler import check_batch, simple_graph

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def to_np(batch):
    return {"ptr": batch.ptr.cpu().numpy(), "idx": batch.idx.cpu().numpy(),
            "sub_to_full": batch.sub_to_full.cpu().numpy(),
            "num_node_in_layer": batch.num_node_in_layer.numpy(),
            "num_edge_in_layer": np.asarray(batch.num_edge_in_layer)}


@pytest.mark.parametrize("fanout,n_seed", [([4], 50), ([5, 3], 64), ([15, 10, 5], 200), ([20, 20], 1)])
def test_sampler_matches_oracle(orc, fanout, n_seed):
    from hiscache import NeighborSampler
    rng = np.random.default_rng(200 + len(fanout))
    indptr, indices = simple_graph(rng, 5000, 30, hubs=5)
    labels = rng.integers(0, 7, size=5000)
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=3, device=DEV)
    for it in range(4):                         # consecutive batches share the node map
        seeds = rng.choice(5000, size=n_seed, replace=False).astype(np.int64)
        print("sampler case", fanout, n_seed, it, flush=True)
        batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
        want = orc.sample_layers(indptr, indices, seeds, fanout, sampler.batch_seed(it))
        got = to_np(batch)
        for k in want:
            np.testing.assert_array_equal(got[k], want[k], err_msg=k)
        np.testing.assert_array_equal(batch.y.cpu().numpy(), labels[seeds])
        check_batch(got, indptr, indices, seeds, fanout)
    # the node map is left clean
    assert int((sampler.node_map != 0x7fffffff).sum()) == 0


def test_sampler_multi_edges_and_isolated_nodes(orc):
    """Adjacency lists with repeated neighbours and nodes without neighbours."""
    from hiscache import NeighborSampler
    rng = np.random.default_rng(210)
    n = 300
    deg = rng.integers(0, 40, size=n)
    deg[:20] = 0
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(deg, out=indptr[1:])
    indices = rng.integers(0, 25, size=int(indptr[-1])).astype(np.int64)     # few targets: many repeats
    sampler = NeighborSampler(indptr, indices, [6, 6], seed=9, device=DEV)
    seeds = np.arange(0, 60, dtype=np.int64)
    batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
    want = orc.sample_layers(indptr, indices, seeds, [6, 6], sampler.batch_seed(0))
    got = to_np(batch)
    for k in want:
        np.testing.assert_array_equal(got[k], want[k], err_msg=k)


@pytest.mark.parametrize("mode", ["launched", "view", "replayed"])
def test_sampled_batch_trains(orc, mode):
    """A batch from the sampler runs through lookup_and_load, the model and update_history; with the view emitted
    with the batch, and with the sampling replayed from HIP graphs (batches pipelined one ahead), the losses
    are the ones of the plain path bit for bit."""
    losses = _train_on_sampled_batches(mode)
    assert all(np.isfinite(losses))
    if mode != "launched":
        assert losses == _train_on_sampled_batches("launched")


def _train_on_sampled_batches(mode):
    from hiscache import HistoryCache, HistorySAGE, NeighborSampler, PinnedFeatureStore, make_config
    rng = np.random.default_rng(220)
    N, Fin, H, C, L = 4000, 32, 48, 5, 3
    indptr, indices = simple_graph(rng, N, 12)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    labels = rng.integers(0, C, size=N)
    sampler = NeighborSampler(indptr, indices, [5, 4, 3], labels=labels, seed=1, device=DEV,
                              emit_view=mode != "launched", replay_slots=3 if mode == "replayed" else 0)
    cfg = make_config(Fin, C, H, L, method="grad", rate=0.6, device=DEV)
    lcm = int(np.lcm(Fin, H))
    cache = HistoryCache(PinnedFeatureStore(feats, device=DEV), cfg, "history_uvm", total_num_node=N,
                         buffer_bytes=600 * lcm * 4, hot_ids=rng.permutation(N).astype(np.int64))
    torch.manual_seed(220)
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
    model.train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2)
    losses = []
    all_seeds = [torch.from_numpy(rng.choice(N, size=100, replace=False)).to(DEV) for _ in range(7)]
    pending = sampler.sample_async(all_seeds[0])
    for it in range(6):
        batch = pending.get()
        pending = sampler.sample_async(all_seeds[it + 1])         # the next batch is drawn while this one trains
        assert (batch.view is None) == (mode == "launched")
        cache.lookup_and_load(batch, L)
        np.testing.assert_array_equal(batch.x.cpu().numpy()[cache.used_masks[0].cpu().numpy()],
                                      feats.numpy()[batch.sub_to_full.cpu().numpy()[cache.used_masks[0].cpu().numpy()]])
        out = model(batch)
        loss = torch.nn.functional.nll_loss(out, batch.y)
        opt.zero_grad()
        loss.backward()
        opt.step()
        cache.update_history(batch, it)
        losses.append(float(loss.detach()))
    pending.get()
    assert cache.header > 0                                   # embeddings were admitted
    return losses


@pytest.mark.parametrize("in_device_memory", [False, True])
def test_training_from_processed_files(tmp_path, in_device_memory):
    """Dataset directory -> feature store (pinned host memory, or the GPU's own), sampler and cache (which reads
    num_nodes.txt and sorted_indices.dat itself) -> a few training iterations."""
    from hiscache import HistoryCache, HistorySAGE, ProcessedDataset, make_config, write_processed
    rng = np.random.default_rng(230)
    N, Fin, H, C, L = 3000, 16, 32, 4, 3
    indptr, indices = simple_graph(rng, N, 10)
    feats = rng.standard_normal((N, Fin)).astype(np.float32)
    write_processed(tmp_path, indptr, indices, feats, hot_ids=rng.permutation(N), labels=rng.integers(0, C, size=N),
                    train_idx=rng.choice(N, size=600, replace=False))
    ds = ProcessedDataset(tmp_path, Fin)
    store = ds.feature_store(device=DEV, in_device_memory=in_device_memory)
    assert store.buffer.is_cuda == in_device_memory
    np.testing.assert_array_equal(store.get(torch.tensor([0, 5, N - 1], device=DEV)).cpu().numpy(),
                                  feats[[0, 5, N - 1]])
    sampler = ds.sampler([4, 3, 2], device=DEV, seed=2, emit_view=True)
    cfg = make_config(Fin, C, H, L, method="grad", rate=0.6, device=DEV, path=str(tmp_path))
    cache = HistoryCache(store, cfg, "history_uvm", buffer_bytes=500 * int(np.lcm(Fin, H)) * 4)
    assert cache.total_num_node == N
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
    model.train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2)
    train = torch.from_numpy(ds.train_idx()).to(DEV)
    pending = sampler.sample_async(train[:100])
    for it in range(5):
        batch = pending.get()
        pending = sampler.sample_async(train[100 * (it + 1): 100 * (it + 2)])     # next batch in flight
        cache.lookup_and_load(batch, L)
        um = cache.used_masks[0].cpu().numpy()
        np.testing.assert_array_equal(batch.x.cpu().numpy()[um], feats[batch.sub_to_full.cpu().numpy()[um]])
        loss = torch.nn.functional.nll_loss(model(batch), batch.y)
        opt.zero_grad()
        loss.backward()
        opt.step()
        cache.update_history(batch, it)
        assert np.isfinite(float(loss.detach()))
    pending.get()
    assert cache.header > 0


def test_recorded_training_from_processed_files(tmp_path):
    """The same pipeline with the sampler replayed from its slots and the iteration recorded and replayed
    (hiscache.RecordedIteration): dataset directory -> store, sampler, HistoryCache from the files, get_model ->
    thirty iterations; the loss falls on labels that a node's own features decide, rows are admitted."""
    from hiscache import HistoryCache, ProcessedDataset, RecordedIteration, get_model, make_config, write_processed
    rng = np.random.default_rng(231)
    N, Fin, H, C, L = 6000, 32, 32, 4, 3
    indptr, indices = simple_graph(rng, N, 10)
    feats = rng.standard_normal((N, Fin)).astype(np.float32)
    labels = feats[:, :C].argmax(1).astype(np.int64)
    write_processed(tmp_path, indptr, indices, feats, hot_ids=rng.permutation(N), labels=labels,
                    train_idx=rng.permutation(N)[:4500])
    ds = ProcessedDataset(tmp_path, Fin)
    store = ds.feature_store(device=DEV)
    sampler = ds.sampler([4, 3, 2], device=DEV, seed=2, emit_view=True, replay_slots=3)
    cfg = make_config(Fin, C, H, L, method="grad", rate=0.6, staleness_thres=5, device=DEV, path=str(tmp_path))
    cache = HistoryCache(store, cfg, "history_uvm", buffer_bytes=1500 * int(np.lcm(Fin, H)) * 4)
    torch.manual_seed(231)
    model = get_model(cfg, cache).to(DEV).train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
    step = RecordedIteration(model, cache, opt, L)
    train = torch.from_numpy(ds.train_idx()).to(DEV)
    pending = sampler.sample_async(train[:150])
    losses, stored = [], 0
    for it in range(1, 30):
        batch = pending.get()
        pending = sampler.sample_async(train[150 * it: 150 * (it + 1)])
        losses.append(float(step(batch, it)))
        stored = max(stored, cache.header)
    pending.get()
    assert all(np.isfinite(losses)) and step.replays >= 20, step.shapes()
    assert np.mean(losses[-5:]) < 0.8 * np.mean(losses[:3]), losses
    assert stored > 0 and cache.glb_iter == 29


@pytest.mark.parametrize("view_edges", [False, True])
def test_replayed_sampling_equals_the_launched_one(orc, view_edges):
    """NeighborSampler(replay_slots=K): the launches of a batch recorded once per slot in a HIP graph and
    replayed for the later batches (new seeds in the slot's array, a new seed key in its pinned word) give the
    sequential statement's batch every time -- ten batches over three slots, with the program's own work and
    synchronisations between the replays --, the emitted view included; a batch with another number of seeds
    takes the ordinary path; a slot's arrays are overwritten when it comes round again."""
    import hiscache_backend as be
    from hiscache import NeighborSampler
    rng = np.random.default_rng(77)
    fanout, n_seed, N = [6, 4], 120, 6000
    indptr, indices = simple_graph(rng, N, 25, hubs=4)
    labels = rng.integers(0, 5, size=N)
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=9, device=DEV, emit_view=True,
                              view_edges=view_edges, replay_slots=3)
    first = None
    for it in range(10):
        n = 37 if it == 6 else n_seed
        seeds = rng.choice(N, size=n, replace=False).astype(np.int64)
        print("replayed sampler batch", it, n, flush=True)
        if it % 4 == 1:                                               # on the caller's (default) stream
            batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
        else:
            pending = sampler.sample_async(torch.from_numpy(seeds).to(DEV))
            x = torch.randn(256, 256, device=DEV)
            (x @ x).sum().item()                                      # eager work and a synchronisation between
            batch = pending.get()
        want = orc.sample_layers(indptr, indices, seeds, fanout, sampler.batch_seed(it))
        got = to_np(batch)
        for k in want:
            np.testing.assert_array_equal(got[k], want[k], err_msg=f"{k} of batch {it}")
        np.testing.assert_array_equal(batch.y.cpu().numpy(), labels[seeds])
        L = len(fanout)
        n_rows, n_src, n_e = int(want["num_node_in_layer"][L - 1]), int(want["num_node_in_layer"][L]), len(want["idx"])
        wp, wr, we = orc.build_transpose(want["ptr"], want["idx"], None, n_src)
        assert batch.view.covers(n_rows, n_src) and batch.view.num_edge == n_e
        np.testing.assert_array_equal(batch.view.ptrT.cpu().numpy(), wp)
        np.testing.assert_array_equal(batch.view.rowT.cpu().numpy()[:n_e], wr)
        if view_edges:
            np.testing.assert_array_equal(batch.view.edgeT.cpu().numpy()[:n_e], we)
        else:
            assert batch.view.edgeT is None
        if it == 0:
            first = (batch, got["idx"].copy())
        if it == 3:                                                   # slot 0 again: the first batch's memory
            assert first[0].idx.data_ptr() == batch.idx.data_ptr()
    assert sum(s is not None and s.graph is not None for s in sampler._slots) == 3
    assert int((sampler.node_map != 0x7fffffff).sum()) == 0
