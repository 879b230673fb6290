"""Recorded iterations: the entry points that read a batch's sizes from device memory, each against its
counterpart that takes them by value, and ``hiscache.RecordedIteration`` over sampled batches of changing
sizes: replayed iterations leave exactly the state that the same padded iterations leave when nothing is
recorded, and that state follows the ordinary (unpadded) loop within fp32 tolerances."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def one(v):
    return torch.tensor([int(v)], dtype=torch.int64, device=DEV)


# ------------------------------------------------------------------------------------------------ entry points
def test_stage_arrays_pads_and_writes_scalars():
    import hiscache_backend as be
    rng = np.random.default_rng(1)
    a64 = rng.integers(-5, 1 << 40, size=1000)
    a32 = rng.integers(-5, 1 << 30, size=777).astype(np.int32)
    f32 = rng.standard_normal((50, 12)).astype(np.float32)
    f16 = rng.standard_normal((40, 6)).astype(np.float16)
    u8 = rng.integers(0, 2, size=333).astype(np.uint8)
    dst = [torch.full((1500,), 9, dtype=torch.int64, device=DEV), torch.full((777,), 9, dtype=torch.int32, device=DEV),
           torch.full((64, 12), 9.0, device=DEV), torch.full((64, 6), 9.0, dtype=torch.float16, device=DEV),
           torch.full((400,), 9, dtype=torch.uint8, device=DEV), torch.full((10,), 9, dtype=torch.int64, device=DEV)]
    scal = torch.zeros(16, dtype=torch.int64, device=DEV)
    be.stage_arrays([(T(a64), dst[0], 1000, -1), (T(a32), dst[1], 500, 7), (T(f32).view(-1), dst[2].view(-1), 50 * 12, 0),
                     (T(f16).view(-1), dst[3].view(-1), 40 * 6, 0), (T(u8), dst[4], 333, 0), (None, dst[5], 0, -3)],
                    scal, [3, -4, 1 << 50])
    np.testing.assert_array_equal(dst[0].cpu().numpy(), np.concatenate([a64, np.full(500, -1)]))
    np.testing.assert_array_equal(dst[1].cpu().numpy(), np.concatenate([a32[:500], np.full(277, 7, np.int32)]))
    np.testing.assert_array_equal(dst[2].cpu().numpy(), np.concatenate([f32, np.zeros((14, 12), np.float32)]))
    np.testing.assert_array_equal(dst[3].cpu().numpy(), np.concatenate([f16, np.zeros((24, 6), np.float16)]))
    np.testing.assert_array_equal(dst[4].cpu().numpy(), np.concatenate([u8, np.zeros(67, np.uint8)]))
    assert (dst[5] == -3).all()
    assert scal[:4].tolist() == [3, -4, 1 << 50, 0]
    be.stage_arrays([], scal, [8])                                   # scalars alone
    assert scal[:2].tolist() == [8, -4]
    with pytest.raises(ValueError):
        be.stage_arrays([(T(a64), dst[0], 2000, 0)])                  # more than the destination holds
    with pytest.raises(ValueError):
        be.stage_arrays([(T(a32), dst[0], 10, 0)])                    # another element type


@pytest.mark.parametrize("n_cap,n,C", [(700, 700, 64), (700, 333, 64), (5000, 4097, 128), (40_000, 25_811, 256),
                                       (300, 2, 8)])
def test_bn_relu_with_the_row_count_on_the_device(n_cap, n, C):
    """Over a matrix of n_cap rows of which n are in use: y and dx of the rows in use and every column statistic
    within fp32 rounding of the call over those n rows alone (the slab partition differs), zeros behind."""
    import hiscache_backend as be
    g = torch.Generator(device=DEV).manual_seed(n_cap + n)
    x = torch.randn(n_cap, C, device=DEV, generator=g) * 2 + 1
    x[n:] = 1e6                                    # what padding rows hold must not matter
    dy = torch.randn(n_cap, C, device=DEV, generator=g)
    dy[n:] = 0                                     # nothing reads a padding row, so no gradient reaches it
    bias, gamma, beta = (torch.randn(C, device=DEV, generator=g) for _ in range(3))
    res = []
    for rows, n_dev in ((n_cap, one(n)), (n, None)):
        xa = x[:rows].clone().requires_grad_(True)
        ga, ba, bi = gamma.clone().requires_grad_(True), beta.clone().requires_grad_(True), bias.clone().requires_grad_(True)
        rm, rv = torch.zeros(C, device=DEV), torch.ones(C, device=DEV)
        cnt = torch.zeros(1, dtype=torch.int64, device=DEV)
        y = be.bias_bn_relu(xa, bi, ga, ba, rm, rv, 0.1, 1e-5, cnt, n_dev)
        y.backward(dy[:rows])
        res.append((y.detach(), xa.grad, ga.grad, ba.grad, rm, rv, int(cnt)))
    pad, ref = res
    assert pad[6] == ref[6] == 1
    assert float(pad[0][n:].abs().max() if n < n_cap else 0) == 0.0
    assert float(pad[1][n:].abs().max() if n < n_cap else 0) == 0.0
    for k, tol in ((0, 1e-4), (1, 2e-4), (2, 2e-4), (3, 2e-4), (4, 1e-5), (5, 1e-5)):
        a, b = pad[k][:n] if k < 2 else pad[k], ref[k][:n] if k < 2 else ref[k]
        scale = float(b.abs().max()) + 1e-12
        assert float((a - b).abs().max()) <= tol * scale, (k, float((a - b).abs().max()), scale)
    if n == n_cap:                                 # all rows in use: the very same launches
        for a, b in zip(pad[:6], ref[:6]):
            assert torch.equal(a, b)


@pytest.mark.parametrize("n_max", [1, 2, 77, 5800, 16_384, 16_385, 100_000])
def test_quantile_with_the_count_on_the_device(n_max):
    """The rank worked out on the device gives the bits of the host's: every n up to the capacity, rates over [0, 1]."""
    import hiscache_backend as be
    from hiscache.util import quantile_threshold
    rng = np.random.default_rng(n_max)
    score = T((np.abs(rng.standard_normal(n_max)) * np.exp(rng.normal(-3, 1.5, size=n_max))).astype(np.float32))
    for n in sorted({1, 2, max(1, n_max // 3), max(1, n_max - 1), n_max}):
        for rate in (0.0, 0.1, 0.5, 0.7, 0.9, 0.999, 1.0):
            got = be.quantile_select_dev(score, one(n), rate)
            want = quantile_threshold(score[:n], rate)
            assert torch.equal(got, want), (n, rate, float(got), float(want))
    # a count outside [1, n_max] is clamped
    assert torch.equal(be.quantile_select_dev(score, one(n_max + 5), 0.5), quantile_threshold(score, 0.5))
    assert torch.equal(be.quantile_select_dev(score, one(0), 0.5), quantile_threshold(score[:1], 0.5))


def test_map_lookup_with_the_count_on_the_device():
    import hiscache_backend as be
    rng = np.random.default_rng(4)
    table = T(rng.integers(-1, 1000, size=5000))
    ids = T(np.concatenate([rng.integers(0, 2500, size=700), np.full(300, -1)]))       # padding ids are -1
    for n_valid in (0, 1, 699, 700, 1000):
        got = be.lookup(table, ids, 2500, n_valid=one(n_valid))
        want = be.lookup(table, ids, 2500)
        want[n_valid:] = -1
        assert torch.equal(got, want)
    with pytest.raises(ValueError):
        be.lookup(table, ids, 0, n_valid=torch.tensor([5], dtype=torch.int32, device=DEV))


def test_ring_lookup_and_admission_with_scalars_on_the_device(orc):
    """hc_ring_lookup_dev / hc_grad_check_dev against the by-value entry points on the same state."""
    import hiscache_backend as be
    rng = np.random.default_rng(9)
    N, cap, H, n_cap, n = 5000, 700, 32, 600, 421
    f2s = np.full(N, -1, np.int64)
    own = rng.choice(N, size=500, replace=False)
    f2s[own] = rng.permutation(cap)[:500]
    s2f = np.full(cap, -1, np.int64)
    s2f[f2s[own]] = own
    checkin = np.where(s2f >= 0, rng.integers(0, 9, size=cap), -1)
    table = rng.standard_normal((cap, H)).astype(np.float32)
    ids = rng.choice(N, size=n_cap, replace=False)
    ids[n:] = -1
    for now in (9, 12):
        slot_v, rows_v = be.ring_lookup(T(f2s), T(ids[:n]), T(table), checkin=T(checkin), now=now, age_limit=5)
        slot_d, rows_d = be.ring_lookup(T(f2s), T(ids), T(table), checkin=T(checkin), now=one(now), age_limit=5,
                                        n_valid=one(n))
        assert torch.equal(slot_d[:n], slot_v) and torch.equal(rows_d[:n], rows_v)
        assert (slot_d[n:] == -1).all() and float(rows_d[n:].abs().max()) == 0.0
    # real ids behind n_valid are padding too
    ids2 = ids.copy()
    ids2[n:] = own[: n_cap - n]
    slot_d, _ = be.ring_lookup(T(f2s), T(ids2), T(table), checkin=T(checkin), now=one(9), age_limit=5, n_valid=one(n))
    assert (slot_d[n:] == -1).all()
    with pytest.raises(ValueError):
        be.ring_lookup(T(f2s), T(ids), T(table), now=one(3))          # the two go together
    # admission: the iteration number from the device, padding kept out by the used mask
    emb = rng.standard_normal((n_cap, H)).astype(np.float32)
    grad = (rng.standard_normal((n_cap, H)) * np.exp(rng.normal(-3, 1.5, size=(n_cap, 1)))).astype(np.float32)
    grad[n:] = 0
    slot = slot_v.cpu().numpy()
    thres = torch.tensor([0.05], device=DEV)
    out = []
    for dev_side in (False, True):
        st = dict(table=T(table), f2s=T(f2s), s2f=T(s2f), chk=T(checkin), header=one(650))
        if dev_side:
            used = torch.arange(n_cap, device=DEV) < one(n)
            mask, _ = be.grad_check(T(grad), T(emb), T(np.concatenate([slot, np.full(n_cap - n, -1)])), T(np.maximum(ids, 0)),
                                    thres, st["table"], st["f2s"], st["s2f"], st["header"], one(17), used=used,
                                    checkin=st["chk"])
            assert not mask[n:].any()
            mask = mask[:n]
        else:
            mask, _ = be.grad_check(T(grad[:n]), T(emb[:n]), T(slot), T(ids[:n]), thres, st["table"], st["f2s"],
                                    st["s2f"], st["header"], 17, checkin=st["chk"])
        out.append((mask, st))
    assert torch.equal(out[0][0], out[1][0]) and 0 < int(out[0][0].sum()) < n
    for k in ("table", "f2s", "s2f", "chk", "header"):
        assert torch.equal(out[0][1][k], out[1][1][k]), k
    assert int((out[1][1]["chk"] == 17).sum()) == int(out[0][0].sum())


# ------------------------------------------------------------------------------------------------ the iteration
def make_world(seed, rate, thres, N, Fin, H, C, L, feats, cached, rows, prefetch_cus=0):
    from hiscache import HistorySAGE, PinnedFeatureStore, RingHistoryCache, make_config
    torch.manual_seed(seed)
    store = PinnedFeatureStore(feats, device=DEV, prefetch_cus=prefetch_cus)
    cache = RingHistoryCache(store, N, Fin, H, capacity=N // 2, num_layers=L, table_dtype=torch.float32, rate=rate,
                             thres=thres, age_limit=3, device=DEV)
    cache.preload(cached.to(DEV), rows.to(DEV))
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device=DEV), cache).to(DEV)
    model.train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
    return cache, model, opt


def state_of(cache, model, opt):
    out = [p.detach().clone() for p in model.parameters()] + [b.clone() for b in model.buffers()]
    out += [cache.table.clone(), cache.full2slot.clone(), cache.slot2full.clone(), cache.checkin.clone(),
            cache._header.clone()]
    for st in opt.state.values():
        out += [st["exp_avg"].clone(), st["exp_avg_sq"].clone(), st["step"].clone()]
    return out


@pytest.mark.parametrize("L,fanout,thres,read_ahead", [(2, [8, 5], None, False), (3, [6, 4, 3], 0.05, False),
                                                        (3, [6, 4, 3], None, True)])
def test_replayed_iterations_equal_the_padded_ones(L, fanout, thres, read_ahead):
    """Twelve sampled batches of changing sizes (some come back after their nodes were admitted; entries go stale
    after three iterations), three twins: replayed, padded but not recorded, and the ordinary loop.  After every
    iteration the first two hold the same bits in every parameter, buffer, optimizer state and cache tensor; with
    ``read_ahead`` the feature rows of the next batch are read beside the replay and corrected inside it."""
    from helpers import power_law_graph
    from hiscache import NeighborSampler, RecordedIteration, backward_on_this_thread, prefer_low_latency_gemm
    N, Fin, H, C, n_seed = 60_000, 64, 64, 7, 300
    rng = np.random.default_rng(5)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=300)      # batch sizes vary by percents
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: N // 4].copy())
    rows = torch.from_numpy(rng.standard_normal((cached.numel(), H)).astype(np.float32) * 0.5)
    prefer_low_latency_gemm()
    args = (0.5, thres, N, Fin, H, C, L, feats, cached, rows)
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=5, device=DEV, emit_view=True)
    gen = torch.Generator(device=DEV).manual_seed(5)
    seeds = [torch.randperm(N, device=DEV, generator=gen)[:n_seed].contiguous() for _ in range(6)]
    order = [0, 1, 2, 0, 3, 1, 4, 0, 5, 2, 3, 0]

    def batches():
        """Every twin trains on batches of its own (a batch object carries its read-ahead)."""
        return [sampler.sample(seeds[k], rng_seed=1000 + k) for k in order]

    worlds = {name: make_world(11, *args) for name in ("recorded", "padded", "plain")}
    rec = RecordedIteration(*[worlds["recorded"][k] for k in (1, 0, 2)], L, step=1.005, round_to=16)
    pad = RecordedIteration(*[worlds["padded"][k] for k in (1, 0, 2)], L, step=1.005, round_to=16, record=False)
    cache_p, model_p, opt_p = worlds["plain"]
    sets = {name: batches() for name in worlds}
    for name in ("ptr", "idx", "sub_to_full"):
        assert all(torch.equal(getattr(a, name), getattr(b, name)) for a, b in zip(sets["recorded"], sets["plain"]))
    losses = {name: [] for name in worlds}
    compute = torch.cuda.Stream()              # the read-ahead runs beside work on a stream of its own
    compute.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(compute):
        for i in range(len(order)):
            it = i + 1
            for name, runner in (("recorded", rec), ("padded", pad)):
                if read_ahead and i + 1 < len(order):
                    runner.prefetch(sets[name][i + 1])
                losses[name].append(float(runner(sets[name][i], it)))
            a, c = state_of(*worlds["recorded"]), state_of(*worlds["padded"])
            same = [bool(torch.equal(x, y)) for x, y in zip(a, c)]
            assert all(same), (it, same)
            assert losses["recorded"][-1] == losses["padded"][-1]
            # the ordinary loop: eager work and synchronisations between the replays
            b = sets["plain"][i]
            cache_p.lookup_and_load(b, L)
            loss = torch.nn.functional.nll_loss(model_p(b), b.y)
            opt_p.zero_grad(set_to_none=True)
            backward_on_this_thread(loss)
            opt_p.step()
            cache_p.update_history(b, it)
            losses["plain"].append(float(loss.detach()))
    torch.cuda.synchronize()
    shapes = rec.shapes()
    assert rec.replays >= len(order) // 3 and sum(1 for v in shapes.values() if v[2]) >= 2, shapes
    assert all((k[2] >= 0) == read_ahead for k, v in shapes.items() if v[2])      # rows read straight into place
    np.testing.assert_allclose(losses["recorded"], losses["plain"], rtol=2e-3)
    for p, q in zip(worlds["recorded"][1].parameters(), model_p.parameters()):
        assert float((p - q).detach().abs().max()) < 2e-2 * float(q.detach().abs().max())
    # the tables hold nearly the same entries (a score next to the threshold may fall on either side)
    a, c = worlds["recorded"][0].full2slot != -1, cache_p.full2slot != -1
    assert int((a != c).sum()) <= max(4, int(0.002 * int(c.sum())))
    assert worlds["recorded"][0].glb_iter == cache_p.glb_iter == len(order)


def test_batches_outside_the_recorded_family_take_the_ordinary_path():
    from helpers import power_law_graph
    from hiscache import NeighborSampler, RecordedIteration, prefer_low_latency_gemm
    N, Fin, H, C, L = 20_000, 32, 32, 5, 2
    rng = np.random.default_rng(8)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=200)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: N // 4].copy())
    rows = torch.from_numpy(rng.standard_normal((cached.numel(), H)).astype(np.float32))
    prefer_low_latency_gemm()
    cache, model, opt = make_world(3, 0.5, None, N, Fin, H, C, L, feats, cached, rows)
    sampler = NeighborSampler(indptr, indices, [6, 4], labels=labels, seed=8, device=DEV, emit_view=True)
    rec = RecordedIteration(model, cache, opt, L, max_records=1)
    gen = torch.Generator(device=DEV).manual_seed(8)
    it = 0
    for n_seed in (200, 200, 200, 57, 200, 400, 200):          # a short last batch of an epoch, a larger one
        it += 1
        loss = rec(sampler.sample(torch.randperm(N, device=DEV, generator=gen)[:n_seed].contiguous()), it)
        assert np.isfinite(float(loss))
    assert cache.glb_iter == it and rec.replays >= 2 and rec.unrecorded >= 3
    assert len(rec.shapes()) == 1


def test_replayed_relational_iterations_equal_the_padded_ones():
    """The relational model (5 relations from node-type ranges, fp16 features and table, the batch's view with edge
    slots, rows read ahead): replayed and padded-but-unrecorded twins hold the same bits after every iteration."""
    from helpers import power_law_graph
    from hiscache import (HistoryRGCN, NeighborSampler, PinnedFeatureStore, RecordedIteration, RingHistoryCache,
                          make_config, prefer_low_latency_gemm)
    n_paper, n_author, n_inst = 20_000, 19_000, 1_000
    N = n_paper + n_author + n_inst
    Fin, H, C, K, L, n_seed, fanout = 64, 64, 9, 5, 2, 200, [10, 6]
    rng = np.random.default_rng(12)
    indptr, indices = power_law_graph(rng, N, 3.0, alpha=2.0, max_degree=300)
    feats = torch.from_numpy(rng.standard_normal((N, Fin), dtype=np.float32).astype(np.float16))
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: N // 3].copy())
    rows = torch.from_numpy((0.5 * rng.standard_normal((cached.numel(), H), dtype=np.float32)).astype(np.float16))
    prefer_low_latency_gemm()

    def world():
        torch.manual_seed(21)
        store = PinnedFeatureStore(feats, device=DEV, out_dtype=torch.float16)
        cache = RingHistoryCache(store, N, Fin, H, capacity=N, num_layers=L, table_dtype=torch.float16, thres=0.05,
                                 age_limit=4, device=DEV)
        cache.preload(cached.to(DEV), rows.to(DEV))
        cfg = make_config(Fin, C, H, L, device=DEV, model_type="rgcn", num_rel=K, name="rmag240m")
        model = HistoryRGCN(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache, num_rel=K, dataset_name="rmag240m",
                            type_bounds=[n_paper, n_paper + n_author],
                            pair_to_rel=[[0, 1, 0], [2, 0, 3], [0, 4, 0]]).to(DEV)
        model.train()
        opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
        return cache, model, opt

    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=12, device=DEV, emit_view=True,
                              view_edges=True)
    gen = torch.Generator(device=DEV).manual_seed(12)
    seeds = [torch.randperm(n_paper, device=DEV, generator=gen)[:n_seed].contiguous() for _ in range(5)]
    order = [0, 1, 2, 0, 3, 1, 4, 0, 2, 3]
    twins = {}
    for name, record in (("recorded", True), ("padded", False)):
        cache, model, opt = world()
        twins[name] = (cache, model, opt, RecordedIteration(model, cache, opt, L, step=1.005, round_to=16, record=record),
                       [sampler.sample(seeds[k], rng_seed=500 + k) for k in order])
    compute = torch.cuda.Stream()
    compute.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(compute):
        for i in range(len(order)):
            losses = []
            for name in ("recorded", "padded"):
                cache, model, opt, runner, bs = twins[name]
                if i + 1 < len(order):
                    runner.prefetch(bs[i + 1])
                losses.append(float(runner(bs[i], i + 1)))
            assert losses[0] == losses[1] and np.isfinite(losses[0])
            a, c = state_of(*twins["recorded"][:3]), state_of(*twins["padded"][:3])
            same = [bool(torch.equal(x, y)) for x, y in zip(a, c)]
            assert all(same), (i, same)
            torch.zeros(1000, device=DEV).sum().item()           # eager work and a synchronisation in between
    rec = twins["recorded"][3]
    shapes = rec.shapes()
    assert rec.replays >= len(order) // 3, shapes
    assert all(k[1] % 10 == 2 and k[2] >= 0 for k, v in shapes.items() if v[2])     # view with edge slots, rows read ahead
    assert int((twins["recorded"][0].full2slot != -1).sum()) > cached.numel()   # rows were admitted


def test_recorded_iterations_with_dropout_train():
    """Dropout inside a recording draws from torch's graph-safe generator: the replays train (the loss falls over
    repeated passes) and stay finite.  (Their random stream is not the eager one, so no twin is compared.)"""
    from helpers import power_law_graph
    from hiscache import (HistorySAGE, NeighborSampler, PinnedFeatureStore, RecordedIteration, RingHistoryCache,
                          make_config, prefer_low_latency_gemm)
    N, Fin, H, C, L = 20_000, 64, 64, 4, 2          # two layers: the cached rows have the input's width
    rng = np.random.default_rng(4)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=200)
    feats_np = rng.standard_normal((N, Fin)).astype(np.float32)
    labels_np = (feats_np[:, :C].argmax(1)).astype(np.int64)            # learnable from a node's own features
    prefer_low_latency_gemm()
    torch.manual_seed(4)
    cache = RingHistoryCache(PinnedFeatureStore(torch.from_numpy(feats_np), device=DEV), N, Fin, H, capacity=N,
                             num_layers=L, table_dtype=torch.float32, rate=0.3, age_limit=2, device=DEV)
    model = HistorySAGE(Fin, H, C, L, 0.3, "CSR_Layer", make_config(Fin, C, H, L, device=DEV, dropout=0.3), cache).to(DEV)
    model.train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
    sampler = NeighborSampler(indptr, indices, [6, 4], labels=torch.from_numpy(labels_np), seed=4, device=DEV,
                              emit_view=True)
    rec = RecordedIteration(model, cache, opt, L)
    gen = torch.Generator(device=DEV).manual_seed(4)
    losses = []
    for it in range(1, 61):
        seeds = torch.randperm(N, device=DEV, generator=gen)[:256].contiguous()
        losses.append(float(rec(sampler.sample(seeds), it)))
    assert all(np.isfinite(losses)) and rec.replays >= 50
    assert np.mean(losses[-10:]) < 0.8 * np.mean(losses[:5]), (losses[:5], losses[-10:])


@pytest.mark.parametrize("read_ahead", [False, True])
def test_replayed_iterations_with_the_flat_cache_equal_the_padded_ones(read_ahead):
    """``HistoryCache`` (the reference's flat buffer with a feature cache in its tail, append-only admission, the
    write position restarted every ``staleness_thres`` iterations): replayed and padded-but-unrecorded twins hold
    the same bits after every iteration, the restart included."""
    from helpers import power_law_graph
    from hiscache import (HistoryCache, HistorySAGE, NeighborSampler, PinnedFeatureStore, RecordedIteration,
                          make_config, prefer_low_latency_gemm)
    N, Fin, H, C, L, n_seed, fanout = 30_000, 64, 64, 6, 3, 200, [6, 4, 3]
    rng = np.random.default_rng(31)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=300)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    hot = rng.permutation(N).astype(np.int64)
    prefer_low_latency_gemm()

    def world():
        torch.manual_seed(17)
        cfg = make_config(Fin, C, H, L, method="grad", rate=0.5, staleness_thres=4, device=DEV)
        cache = HistoryCache(PinnedFeatureStore(feats, device=DEV), cfg, "history_uvm", total_num_node=N,
                             buffer_bytes=6000 * 64 * 4, hot_ids=hot)
        model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
        model.train()
        opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
        return cache, model, opt

    def state(cache, model, opt):
        out = [p.detach().clone() for p in model.parameters()] + [b.clone() for b in model.buffers()]
        out += [cache.buffer.clone(), cache.full2embed.clone(), cache.embed2full.clone(), cache._header.clone(),
                cache._num_stored.clone()]
        for st in opt.state.values():
            out += [st["exp_avg"].clone(), st["exp_avg_sq"].clone()]
        return out

    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=31, device=DEV, emit_view=True)
    gen = torch.Generator(device=DEV).manual_seed(31)
    seeds = [torch.randperm(N, device=DEV, generator=gen)[:n_seed].contiguous() for _ in range(5)]
    order = [0, 1, 2, 0, 3, 1, 4, 0, 2, 3, 1, 0]
    twins = {}
    for name, record in (("recorded", True), ("padded", False)):
        cache, model, opt = world()
        twins[name] = (cache, model, opt, RecordedIteration(model, cache, opt, L, step=1.005, round_to=16, record=record),
                       [sampler.sample(seeds[k], rng_seed=700 + k) for k in order])
    compute = torch.cuda.Stream()
    compute.wait_stream(torch.cuda.current_stream())
    admitted = []
    with torch.cuda.stream(compute):
        for i in range(len(order)):
            losses = []
            for name in ("recorded", "padded"):
                cache, model, opt, runner, bs = twins[name]
                if read_ahead and i + 1 < len(order):
                    runner.prefetch(bs[i + 1])
                losses.append(float(runner(bs[i], i + 1)))
            assert losses[0] == losses[1] and np.isfinite(losses[0])
            a, c = state(*twins["recorded"][:3]), state(*twins["padded"][:3])
            same = [bool(torch.equal(x, y)) for x, y in zip(a, c)]
            assert all(same), (i, same)
            admitted.append(twins["recorded"][0].header)
    rec = twins["recorded"][3]
    assert rec.replays >= len(order) // 3, rec.shapes()
    assert admitted[2] > 0 and admitted[3] < admitted[2]          # iteration 4 restarted the write position
    assert twins["recorded"][0].glb_iter == len(order)


def test_padded_layers_aggregate_nothing_behind_their_real_rows():
    """In a padded batch the rows between a layer's real count and its padded count are real rows of the next hop:
    their sources lie behind the layer's input.  Every layer gets row offsets of its own that leave them empty, so
    its aggregation output is zero there (it read nothing), whatever lies behind the input in memory."""
    from helpers import power_law_graph
    from hiscache import NeighborSampler, RecordedIteration, prefer_low_latency_gemm
    N, Fin, H, C, L = 40_000, 64, 64, 5, 3
    rng = np.random.default_rng(77)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=300)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32) + 3.0)     # no zero rows by chance
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: N // 4].copy())
    rows = torch.from_numpy(rng.standard_normal((cached.numel(), H)).astype(np.float32) + 3.0)
    prefer_low_latency_gemm()
    cache, model, opt = make_world(5, 0.5, None, N, Fin, H, C, L, feats, cached, rows)
    sampler = NeighborSampler(indptr, indices, [6, 4, 3], labels=labels, seed=77, device=DEV, emit_view=True)
    rec = RecordedIteration(model, cache, opt, L, step=1.3, round_to=512, record=False)   # generous padding
    gen = torch.Generator(device=DEV).manual_seed(77)
    seen = []
    hooks = [conv.register_forward_hook(lambda mod, args, out: seen.append(out[1].detach().clone()))
             for conv in model.convs]
    for it in (1, 2):
        batch = sampler.sample(torch.randperm(N, device=DEV, generator=gen)[:250].contiguous())
        nnl = [int(v) for v in batch.num_node_in_layer]
        seen.clear()
        loss = rec(batch, it)
        assert np.isfinite(float(loss))
        (caps, _, _, _), = rec.shapes().values()
        assert caps[1] > nnl[1] and caps[2] > nnl[2]
        for i, agg in enumerate(seen):                       # layer i produces the rows of hop L - 1 - i
            k = L - 1 - i
            assert agg.shape[0] == caps[k]
            assert float(agg[nnl[k]:].abs().max() if caps[k] > nnl[k] else 0.0) == 0.0, (it, i)
            assert float(agg[: nnl[k]].abs().sum()) > 0.0   # (while the real rows were aggregated)
    for h in hooks:
        h.remove()
    for p in model.parameters():
        assert torch.isfinite(p).all()


@pytest.mark.parametrize("relational", [False, True])
def test_padded_iterations_pass_the_device_side_input_checks(monkeypatch, relational):
    """With the library's debugging switch on, every aggregation call of a padded iteration first has its row
    offsets and neighbour ids checked on the device against the layer's input rows, and every backward over the
    batch's view has the view's columns, rows and edge slots checked: a padded layer that reached behind its
    input would be reported here instead of reading there."""
    import hiscache_backend as be
    from helpers import power_law_graph
    from hiscache import (HistoryRGCN, NeighborSampler, PinnedFeatureStore, RecordedIteration, RingHistoryCache,
                          make_config, prefer_low_latency_gemm)
    N, Fin, H, C, L = 40_000, 64, 64, 5, 3
    rng = np.random.default_rng(78)
    indptr, indices = power_law_graph(rng, N, 4.0, alpha=2.0, max_degree=300)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: N // 4].copy())
    rows = torch.from_numpy(rng.standard_normal((cached.numel(), H)).astype(np.float32))
    prefer_low_latency_gemm()
    if relational:
        torch.manual_seed(6)
        store = PinnedFeatureStore(feats, device=DEV)
        cache = RingHistoryCache(store, N, Fin, H, capacity=N // 2, num_layers=L, table_dtype=torch.float32,
                                 thres=0.05, age_limit=3, device=DEV)
        cache.preload(cached.to(DEV), rows.to(DEV))
        cfg = make_config(Fin, C, H, L, device=DEV, model_type="rgcn", num_rel=5, name="rmag240m")
        model = HistoryRGCN(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache, num_rel=5, dataset_name="rmag240m",
                            type_bounds=[N // 2, N - 1000], pair_to_rel=[[0, 1, 0], [2, 0, 3], [0, 4, 0]]).to(DEV)
        model.train()
        opt = torch.optim.Adam(model.parameters(), lr=1e-2, fused=True, capturable=True)
    else:
        cache, model, opt = make_world(6, 0.5, None, N, Fin, H, C, L, feats, cached, rows)
    sampler = NeighborSampler(indptr, indices, [6, 4, 3], labels=labels, seed=78, device=DEV, emit_view=True,
                              view_edges=relational)
    rec = RecordedIteration(model, cache, opt, L, step=1.3, round_to=512, record=False)
    gen = torch.Generator(device=DEV).manual_seed(78)
    monkeypatch.setattr(be, "CHECK_INPUTS", True)
    checked = []
    real_check = be.check_csr
    monkeypatch.setattr(be, "check_csr", lambda *a: (checked.append(a[2:]), real_check(*a))[1])
    for it in (1, 2, 3):
        batch = sampler.sample(torch.randperm(N // 2, device=DEV, generator=gen)[:250].contiguous())
        assert np.isfinite(float(rec(batch, it)))
    (caps, _, _, _), = rec.shapes().values()
    # every layer's forward was checked against ITS input rows, every backward over the view against its sources
    assert {(caps[k], caps[k + 1]) for k in range(L)} <= set(checked) or relational
    assert len(checked) >= 3 * (2 * L - 1)            # (the first layer hands no gradient to the features)
    # the check itself reports rows whose sources lie behind the input it is told of
    b = rec._records[next(iter(rec._records))].batch
    with pytest.raises(ValueError, match="neighbour ids outside"):
        real_check(b.ptr, b.idx, caps[L - 1], caps[L - 1])
