"""The feature matrix in two tiers (copies of the hot rows in device memory, everything in pinned host memory):
whatever is read through the tiers equals, bit for bit, what the same request reads from the host matrix alone --
the two launches by themselves, the store's ``get`` / ``masked_get`` / ``prefetch`` + ``take``, a dataset directory
with its hotness order, and training (ordinary and recorded) on a tiered store against a plain one."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def host_matrix(rng, n, F, dtype):
    a = torch.from_numpy(rng.standard_normal((n, F)).astype(np.float32)).to(TORCH[dtype])
    pinned = torch.empty(a.shape, dtype=a.dtype, pin_memory=True)
    pinned.copy_(a)
    return pinned


@pytest.mark.parametrize("src_dtype,out_dtype", [("f32", "f32"), ("f16", "f16"), ("f16", "f32"), ("bf16", "f32"),
                                                 ("f32", "f16")])
@pytest.mark.parametrize("N,F,n,hot_share,masked", [(5000, 128, 3000, 0.3, True), (5000, 100, 1111, 0.5, True),
                                                    (4000, 768, 700, 0.2, False), (300, 1, 65, 0.5, True),
                                                    (300, 6, 64, 0.0, True), (300, 8, 63, 1.0, False),
                                                    (50, 4, 1, 0.5, False), (20_000, 128, 40_000, 0.4, True)])
def test_two_launches_equal_the_plain_gather(src_dtype, out_dtype, N, F, n, hot_share, masked):
    import hiscache_backend as be
    rng = np.random.default_rng(N + F + n)
    src = host_matrix(rng, N, F, src_dtype)
    k = int(N * hot_share)
    hot_ids = torch.from_numpy(rng.permutation(N)[:k].copy()).to(DEV)
    slot = torch.full((N,), -1, dtype=torch.int32, device=DEV)
    slot[hot_ids] = torch.arange(k, dtype=torch.int32, device=DEV)
    hot = src.to(DEV)[hot_ids].contiguous() if k else torch.empty((0, F), dtype=src.dtype, device=DEV)
    ids_np = rng.integers(0, N, size=n)
    if n > 10:                                   # ids that address from the end, ids outside the matrix
        ids_np[1], ids_np[2], ids_np[3], ids_np[4] = -1, -N, N, -N - 1
    ids = torch.from_numpy(ids_np).to(DEV)
    mask = torch.from_numpy(rng.random(n) < 0.6).to(DEV) if masked else None
    want = be.gather_rows(src, ids, mask=mask, out_dtype=TORCH[out_dtype])
    # (the same matrix in device memory is gathered several rows per wave: the same rows)
    assert torch.equal(be.gather_rows(src.to(DEV), ids, mask=mask, out_dtype=TORCH[out_dtype]), want)

    out = torch.full((n, F), 7.0, dtype=TORCH[out_dtype], device=DEV)
    rows, cold = be.gather_rows_hot(hot, slot, ids, mask=mask, out=out)
    assert rows.data_ptr() == out.data_ptr()
    # which rows were left for the other launch: asked for, inside the matrix, without a device copy
    wrapped = np.where(ids_np < 0, ids_np + N, ids_np)
    inside = (wrapped >= 0) & (wrapped < N)
    take = inside & (mask.cpu().numpy() if masked else np.ones(n, bool))
    slot_np = slot.cpu().numpy()
    expect_cold = take & (slot_np[np.where(inside, wrapped, 0)] < 0)
    assert np.array_equal(cold.cpu().numpy().astype(bool), expect_cold)
    untouched = torch.from_numpy(expect_cold).to(DEV)
    assert bool((out[untouched] == 7.0).all())                     # left alone by the first launch
    assert torch.equal(out[~untouched], want[~untouched])
    before = out.clone()
    be.gather_rows_flagged(src, ids, cold, out)
    assert torch.equal(out, want)
    assert torch.equal(out[~untouched], before[~untouched])        # the second launch wrote its own rows only
    # the host matrix stored under other row numbers (two id arrays) and a device-memory source
    shift = (ids + 17) % N
    out2 = before.clone()
    be.gather_rows_flagged(src.to(DEV), shift, cold, out2)
    assert torch.equal(out2[untouched], be.gather_rows(src, shift, out_dtype=TORCH[out_dtype])[untouched])
    # a flagged row whose source row does not exist is cleared
    if n > 10:
        bad = ids.clone()
        flagged = torch.nonzero(cold).view(-1)
        if flagged.numel():
            bad[flagged[0]] = N + 5
            out3 = before.clone()
            be.gather_rows_flagged(src, bad, cold, out3)
            assert float(out3[flagged[0]].float().abs().max()) == 0.0


def test_argument_checks():
    import hiscache_backend as be
    hot = torch.zeros((4, 8), device=DEV)
    slot = torch.full((10,), -1, dtype=torch.int32, device=DEV)
    ids = torch.arange(5, device=DEV)
    with pytest.raises(ValueError):
        be.gather_rows_hot(hot, slot.long(), ids)                  # the map is int32
    with pytest.raises(ValueError):
        be.gather_rows_hot(hot, slot, ids, out=torch.zeros((5, 9), device=DEV))
    with pytest.raises(RuntimeError):
        be.gather_rows_flagged(torch.zeros((10, 8)), ids, torch.ones(5, dtype=torch.uint8, device=DEV),
                               torch.zeros((5, 8), device=DEV))    # pageable host memory
    with pytest.raises(ValueError):
        be.gather_rows_flagged(hot, ids, torch.ones(4, dtype=torch.uint8, device=DEV), torch.zeros((5, 8), device=DEV))
    out, cold = be.gather_rows_hot(hot, slot, ids[:0])
    assert out.shape == (0, 8) and cold.numel() == 0


@pytest.mark.parametrize("prefetch_cus", [0, 16])
def test_store_reads_through_the_tiers_equal_the_plain_store(prefetch_cus):
    from hiscache import PinnedFeatureStore
    rng = np.random.default_rng(3)
    N, F = 30_000, 128
    src = host_matrix(rng, N, F, "f32")
    plain = PinnedFeatureStore(src, device=DEV)
    tiered = PinnedFeatureStore(src, device=DEV, prefetch_cus=prefetch_cus,
                                hot_ids=torch.from_numpy(rng.permutation(N)[: N // 3].copy()))
    assert tiered.hot_rows.shape == (N // 3, F) and tiered.hot_rows.is_cuda
    compute = torch.cuda.Stream()
    compute.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(compute):
        for trial in range(4):
            ids = torch.from_numpy(rng.integers(0, N, size=9000)).to(DEV)
            guess = torch.from_numpy(rng.random(9000) < 0.5).to(DEV)
            need = torch.from_numpy(rng.random(9000) < 0.5).to(DEV)
            assert torch.equal(tiered.get(ids), plain.get(ids))
            assert torch.equal(tiered.masked_get(ids, need), plain.masked_get(ids, need))
            cold = int(tiered.last_cold.sum())
            assert 0 < cold < int(need.sum())                      # some rows came from each tier
            out = torch.full((9000, F), 3.0, device=DEV) if trial % 2 else None
            handle = tiered.prefetch(ids, guess, out=out)
            torch.zeros(1 << 20, device=DEV).sum()                 # work beside the read
            rows = tiered.take(handle, need)
            assert out is None or rows.data_ptr() == out.data_ptr()
            assert torch.equal(rows, plain.masked_get(ids, need))
            rows_async, ev = tiered.masked_get_async(ids, need)
            tiered.join(ev)
            assert torch.equal(rows_async, plain.masked_get(ids, need))
    torch.cuda.synchronize()
    # the read-ahead stream goes while tensors that it filled are alive; they stay valid and are freed later
    keep = rows.clone()
    tiered.close()
    assert torch.equal(rows, keep)
    handle = tiered.prefetch(ids, guess)                           # (a new stream is made on demand)
    assert torch.equal(tiered.take(handle, need), plain.masked_get(ids, need))
    tiered.close()
    del rows, handle, out, rows_async
    with pytest.raises(ValueError):
        PinnedFeatureStore(src.to(DEV), device=DEV, hot_ids=torch.arange(10))     # all of it is in device memory
    with pytest.raises(ValueError):
        PinnedFeatureStore(src, device=DEV, hot_ids=torch.tensor([N]))


def test_dataset_directory_keeps_its_hottest_rows_on_the_device(tmp_path):
    from helpers import power_law_graph
    from hiscache import ProcessedDataset
    from hiscache.dataset import write_processed
    rng = np.random.default_rng(4)
    N, F = 3000, 16
    indptr, indices = power_law_graph(rng, N, 3.0, alpha=2.0, max_degree=50)
    feats = rng.standard_normal((N, F)).astype(np.float32)
    order = rng.permutation(N)                                     # hottest last
    write_processed(tmp_path, indptr, indices, feats, hot_ids=order)
    ds = ProcessedDataset(tmp_path, feature_dim=F)
    store = ds.feature_store(device=DEV, hot_rows=500)
    slot = store.hot_slot.cpu().numpy()
    assert np.array_equal(np.sort(np.nonzero(slot >= 0)[0]), np.sort(order[-500:]))
    assert np.array_equal(store.hot_rows.cpu().numpy()[slot[order[-500:]]], feats[order[-500:]])
    ids = torch.from_numpy(rng.integers(0, N, size=2000)).to(DEV)
    assert np.array_equal(store.get(ids).cpu().numpy(), feats[ids.cpu().numpy()])
    assert int(store.last_cold.sum()) == int((slot[ids.cpu().numpy()] < 0).sum())


@pytest.mark.parametrize("recorded", [False, True])
def test_training_on_a_tiered_store_equals_training_on_a_plain_one(recorded):
    """Twins that differ only in the store (a third of the rows with a device copy, rows read one batch ahead):
    the same bits in every parameter, optimizer state and cache tensor after every iteration, in the ordinary
    loop and in the recorded one."""
    from helpers import power_law_graph
    from hiscache import (HistorySAGE, NeighborSampler, PinnedFeatureStore, RecordedIteration, RingHistoryCache,
                          backward_on_this_thread, make_config, prefer_low_latency_gemm)
    N, Fin, H, C, L, n_seed = 50_000, 64, 64, 6, 3, 250
    rng = np.random.default_rng(9)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=300)
    feats = host_matrix(rng, N, Fin, "f32")
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: N // 4].copy())
    rows = torch.from_numpy(rng.standard_normal((cached.numel(), H)).astype(np.float32) * 0.5)
    in_degree = np.bincount(indices, minlength=N)
    hot_ids = torch.from_numpy(np.argsort(in_degree, kind="stable")[-N // 3:].copy())
    prefer_low_latency_gemm()

    def world(tiers):
        torch.manual_seed(2)
        store = PinnedFeatureStore(feats, device=DEV, prefetch_cus=16, hot_ids=hot_ids if tiers else None)
        cache = RingHistoryCache(store, N, Fin, H, capacity=N // 2, num_layers=L, table_dtype=torch.float32,
                                 thres=0.05, age_limit=3, device=DEV)
        cache.preload(cached.to(DEV), rows.to(DEV))
        model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device=DEV), cache).to(DEV)
        model.train()
        opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
        run = RecordedIteration(model, cache, opt, L, step=1.01, round_to=32) if recorded else None
        return store, cache, model, opt, run

    sampler = NeighborSampler(indptr, indices, [6, 4, 3], labels=labels, seed=9, device=DEV, emit_view=True)
    gen = torch.Generator(device=DEV).manual_seed(9)
    seeds = [torch.randperm(N, device=DEV, generator=gen)[:n_seed].contiguous() for _ in range(4)]
    order = [0, 1, 2, 0, 3, 1, 2, 0, 3, 1]
    twins = {name: world(name == "tiered") for name in ("tiered", "plain")}
    sets = {name: [sampler.sample(seeds[k], rng_seed=70 + k) for k in order] for name in twins}

    def state(w):
        _, cache, model, opt, _ = w
        out = [p.detach().clone() for p in model.parameters()] + [b.clone() for b in model.buffers()]
        out += [cache.table.clone(), cache.full2slot.clone(), cache.checkin.clone(), cache._header.clone()]
        for st in opt.state.values():
            out += [st["exp_avg"].clone(), st["exp_avg_sq"].clone()]
        return out

    compute = torch.cuda.Stream()
    compute.wait_stream(torch.cuda.current_stream())
    cold_rows = 0
    with torch.cuda.stream(compute):
        for i in range(len(order)):
            losses = []
            for name in ("tiered", "plain"):
                store, cache, model, opt, run = twins[name]
                b = sets[name][i]
                if recorded:
                    if i + 1 < len(order):
                        run.prefetch(sets[name][i + 1])
                    losses.append(float(run(b, i + 1)))
                else:
                    cache.lookup_and_load(b, L)
                    if i + 1 < len(order):
                        cache.prefetch(sets[name][i + 1], speculative=True, num_layer=L)
                    loss = torch.nn.functional.nll_loss(model(b), b.y)
                    opt.zero_grad(set_to_none=True)
                    backward_on_this_thread(loss)
                    opt.step()
                    cache.update_history(b, i + 1)
                    losses.append(float(loss.detach()))
            assert losses[0] == losses[1] and np.isfinite(losses[0])
            same = [bool(torch.equal(x, y)) for x, y in zip(state(twins["tiered"]), state(twins["plain"]))]
            assert all(same), (i, same)
            cold_rows += int(twins["tiered"][0].last_cold.sum())
    torch.cuda.synchronize()
    assert cold_rows > 0
    if recorded:
        assert twins["tiered"][4].replays >= 3, twins["tiered"][4].shapes()


def test_the_flat_cache_on_a_tiered_store_equals_the_flat_cache_on_a_plain_one():
    """``HistoryCache`` (a feature cache of its own in the buffer's tail) over a store with hot rows: what its
    feature cache does not hold comes through the store's two tiers; twins hold the same bits after every
    iteration, with the next batch's rows read ahead."""
    from helpers import power_law_graph
    from hiscache import (HistoryCache, HistorySAGE, NeighborSampler, PinnedFeatureStore, backward_on_this_thread,
                          make_config, prefer_low_latency_gemm)
    N, Fin, H, C, L, n_seed, fanout = 30_000, 64, 64, 6, 3, 200, [6, 4, 3]
    rng = np.random.default_rng(41)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=300)
    feats = host_matrix(rng, N, Fin, "f32")
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    hot = rng.permutation(N).astype(np.int64)                      # hottest last
    prefer_low_latency_gemm()

    def world(tiers):
        torch.manual_seed(17)
        cfg = make_config(Fin, C, H, L, method="grad", rate=0.5, staleness_thres=4, device=DEV)
        # the store's device copies: the 9 000 hottest rows, of which the cache's own tail holds a part
        store = PinnedFeatureStore(feats, device=DEV, prefetch_cus=16,
                                   hot_ids=torch.from_numpy(hot[-9000:].copy()) if tiers else None)
        cache = HistoryCache(store, cfg, "history_uvm", total_num_node=N, buffer_bytes=6000 * 64 * 4, hot_ids=hot)
        model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
        model.train()
        return store, cache, model, torch.optim.Adam(model.parameters(), lr=1e-2, fused=True)

    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=41, device=DEV, emit_view=True)
    gen = torch.Generator(device=DEV).manual_seed(41)
    seeds = [torch.randperm(N, device=DEV, generator=gen)[:n_seed].contiguous() for _ in range(4)]
    order = [0, 1, 2, 0, 3, 1, 2, 0]
    twins = {name: world(name == "tiered") for name in ("tiered", "plain")}
    sets = {name: [sampler.sample(seeds[k], rng_seed=900 + k) for k in order] for name in twins}
    compute = torch.cuda.Stream()
    compute.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(compute):
        for i in range(len(order)):
            xs, losses = [], []
            for name in ("tiered", "plain"):
                store, cache, model, opt = twins[name]
                b = sets[name][i]
                cache.lookup_and_load(b, L)
                xs.append(b.x.clone())
                if i + 1 < len(order):
                    cache.prefetch(sets[name][i + 1], speculative=True, num_layer=L)
                loss = torch.nn.functional.nll_loss(model(b), b.y)
                opt.zero_grad(set_to_none=True)
                backward_on_this_thread(loss)
                opt.step()
                cache.update_history(b, i + 1)
                losses.append(float(loss.detach()))
            assert torch.equal(xs[0], xs[1]), i
            assert losses[0] == losses[1] and np.isfinite(losses[0])
            a, c = twins["tiered"][1], twins["plain"][1]
            assert torch.equal(a.buffer, c.buffer) and torch.equal(a.full2embed, c.full2embed)
            for p, q in zip(twins["tiered"][2].parameters(), twins["plain"][2].parameters()):
                assert torch.equal(p, q)
    torch.cuda.synchronize()
    assert twins["tiered"][0].last_cold is not None and int(twins["tiered"][0].last_cold.sum()) > 0


def test_streams_chosen_by_measurement():
    """The probes behind the loop's long-lived streams.  What they find depends on the machine (how many hardware
    queues, who else uses them), so their verdicts are printed, not asserted -- except that a stream shares a queue
    with itself; what is asserted is that the streams they return are new ones and work: the store's choice of the
    stream that runs beside its reads, the sampler's stream."""
    import hiscache_backend as be
    from hiscache import NeighborSampler, PinnedFeatureStore
    cur = torch.cuda.current_stream()
    assert be.streams_share_queue(cur, cur)
    a = be.stream_apart_from([cur])
    b = be.stream_apart_from([cur, a])
    assert len({cur.cuda_stream, a.cuda_stream, b.cuda_stream}) == 3
    print("shared queues: a/cur", be.streams_share_queue(a, cur), "b/cur", be.streams_share_queue(b, cur),
          "b/a", be.streams_share_queue(b, a), flush=True)
    rng = np.random.default_rng(3)
    feats = torch.from_numpy(rng.standard_normal((50_000, 64)).astype(np.float32)).pin_memory()
    store = PinnedFeatureStore(feats, device=DEV, prefetch_cus=16)
    quiet = store.quiet_stream(candidates=3, rows=20_000, apart_from=[a])
    assert quiet.cuda_stream not in (cur.cuda_stream, a.cuda_stream) and store.quiet_stream_ms > 0
    ids = torch.from_numpy(rng.integers(0, 50_000, size=3000)).to(DEV)
    handle = store.prefetch(ids)
    with torch.cuda.stream(quiet):
        rows = store.take(handle)
        total = rows.sum()
    quiet.synchronize()
    assert torch.equal(rows.cpu(), feats[ids.cpu()]) and torch.isfinite(total)
    store.close()
    plain = PinnedFeatureStore(feats, device=DEV)                      # no stream of limited width: only kept apart
    assert plain.quiet_stream(apart_from=[a]).cuda_stream not in (cur.cuda_stream, a.cuda_stream)
    indptr = np.arange(0, 5001 * 4, 4, dtype=np.int64)
    sampler = NeighborSampler(indptr, rng.integers(0, 5000, size=20000).astype(np.int64), [3, 2], seed=1, device=DEV)
    assert sampler.stream() is sampler.stream() and sampler.stream().cuda_stream != cur.cuda_stream
    batch = sampler.sample_async(torch.arange(100, device=DEV)).get()
    assert int(batch.num_node_in_layer[0]) == 100
