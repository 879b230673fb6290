"""Hotness orders (``hiscache.hotness``): the three metrics against brute force, the cached set's threshold rule, the
file round trip, the embedding-cache simulation against its loops; on the GPU the access counts of sampled batches and what the hottest rows buy a tiered store."""
import numpy as np
import pytest
import torch


def small_graph(rng, n=300, deg=6):
    indptr = np.zeros(n + 1, np.int64)
    indptr[1:] = np.cumsum(rng.integers(0, 2 * deg, size=n))
    indices = rng.integers(0, n, size=indptr[-1]).astype(np.int64)
    return indptr, indices


def test_degree_and_pagerank_against_brute_force():
    from hiscache.hotness import degree_metric, pagerank_metric
    rng = np.random.default_rng(1)
    indptr, indices = small_graph(rng)
    n = len(indptr) - 1
    assert np.array_equal(degree_metric(indptr).numpy(), np.diff(indptr))
    train = rng.choice(n, size=40, replace=False)
    got = pagerank_metric(indptr, indices, train, num_iter=4, damping=0.95).numpy()
    # the rule written out with a dense adjacency matrix in fp64
    A = np.zeros((n, n))
    for r in range(n):
        for j in indices[indptr[r]:indptr[r + 1]]:
            A[r, j] += 1.0
    deg = np.maximum(np.diff(indptr), 1).astype(np.float64)
    score = np.full(n, 1.0 / n)
    score[train] = (n / len(train)) / n
    for _ in range(4):
        score = score / deg
        score = score + A @ score
        score = (1 - 0.95) / n + 0.95 * score
    np.testing.assert_allclose(got, score, rtol=2e-5)
    # no rounds: the start vector; nodes without neighbours keep a finite score
    np.testing.assert_allclose(pagerank_metric(indptr, indices, train, 0).numpy()[train], 1.0 / len(train), rtol=1e-6)
    assert np.isfinite(got).all()


def test_order_cache_map_hit_rate_and_file(tmp_path):
    from types import SimpleNamespace
    from hiscache import ProcessedDataset
    from hiscache.hotness import feature_cache_hit_rate, get_cache_map, hotness_order, write_hotness_order
    metric = torch.tensor([5, 0, 9, 5, 1, 9, 2])
    order = hotness_order(metric)
    assert order.tolist() == [1, 4, 6, 0, 3, 2, 5]                  # ascending metric, ties by id: hottest last
    # the cached set: every node whose metric reaches the metric of the cache_num-th hottest (ties all taken)
    assert get_cache_map(metric, 2).tolist() == [True, False, True, True, False, True, False]   # threshold 5
    assert get_cache_map(metric, 1).tolist() == [False, False, True, False, False, True, False]
    assert not get_cache_map(metric, 0).any() and get_cache_map(metric, 7).all()
    status = get_cache_map(metric, 1)
    batches = [SimpleNamespace(sub_to_full=torch.tensor([2, 5, 0])), SimpleNamespace(sub_to_full=torch.tensor([1, 2]))]
    assert feature_cache_hit_rate(status, batches) == (3 / 5, 3, 5)
    assert feature_cache_hit_rate(status, []) == (0.0, 0, 0)
    with open(tmp_path / "x", "w"):
        pass
    p = write_hotness_order(tmp_path, order)
    assert np.array_equal(np.fromfile(p, dtype=np.int64), order.numpy())
    (tmp_path / "processed" / "num_nodes.txt").write_text("7\n")
    assert np.array_equal(ProcessedDataset(tmp_path, 4).hot_ids(), order.numpy())


@pytest.mark.gpu
def test_access_counts_of_sampled_batches_and_what_the_hot_rows_serve():
    """``profile_metric`` counts a node once per batch that holds it; the rows of the most accessed nodes, kept in
    device memory, serve more of the next epoch's reads than the same number of rows chosen by degree or at random."""
    from helpers import power_law_graph
    from hiscache import NeighborSampler, PinnedFeatureStore
    from hiscache.hotness import (degree_metric, feature_cache_hit_rate, get_cache_map, hotness_order,
                                  profile_metric)
    DEV = "cuda:0"
    rng = np.random.default_rng(5)
    N, F = 40_000, 32
    d_ptr, d_idx = power_law_graph(rng, N, 3.0, alpha=1.8, max_degree=1000)
    # undirected, as the dataset directories hold their graphs: a node's degree then counts its incoming edges too
    src = np.repeat(np.arange(N), np.diff(d_ptr))
    both_src, both_dst = np.concatenate([src, d_idx]), np.concatenate([d_idx, src])
    indptr = np.zeros(N + 1, np.int64)
    np.cumsum(np.bincount(both_src, minlength=N), out=indptr[1:])
    indices = both_dst[np.argsort(both_src, kind="stable")].astype(np.int64)
    sampler = NeighborSampler(indptr, indices, [5, 4, 3], seed=5, device=DEV)
    train = torch.from_numpy(rng.choice(N, size=4000, replace=False)).to(DEV)
    gen = torch.Generator(device=DEV).manual_seed(5)
    metric = profile_metric(sampler, train, 250, num_epochs=2, generator=gen)
    assert metric.shape == (N,) and int(metric.max()) <= 2 * 16 and int(metric[train].min()) >= 2
    # by hand for one epoch of one batch: every node of the batch counted once
    one = profile_metric(NeighborSampler(indptr, indices, [5, 4, 3], seed=9, device=DEV), train[:250], 250)
    assert int(one.sum()) == int((one > 0).sum()) and int(one[train[:250]].min()) == 1
    # the next epoch's batches against three cached sets of the same size
    k = N // 10
    batches = [sampler.sample(train[lo:lo + 250].contiguous()) for lo in range(0, 4000, 250)]
    by_access = feature_cache_hit_rate(get_cache_map(metric, k), batches)[0]
    by_degree = feature_cache_hit_rate(get_cache_map(degree_metric(torch.from_numpy(indptr)).to(DEV), k), batches)[0]
    random_set = torch.zeros(N, dtype=torch.bool, device=DEV)
    random_set[torch.from_numpy(rng.permutation(N)[:k].copy()).to(DEV)] = True
    at_random = feature_cache_hit_rate(random_set, batches)[0]
    assert by_access > 2 * at_random and by_degree > 1.5 * at_random and by_access > 0.9 * by_degree, \
        (by_access, by_degree, at_random)
    # the store with the head of that order as its hot rows: the rows that cross the host link are the misses
    feats = torch.from_numpy(rng.standard_normal((N, F)).astype(np.float32))
    store = PinnedFeatureStore(feats, device=DEV, hot_ids=hotness_order(metric)[-k:])
    b = batches[0]
    assert torch.equal(store.get(b.sub_to_full).cpu(), feats[b.sub_to_full.cpu()])
    hot = torch.zeros(N, dtype=torch.bool, device=DEV)
    hot[hotness_order(metric)[-k:]] = True
    assert int(store.last_cold.sum()) == int((~hot[b.sub_to_full]).sum())
    # the embedding-cache simulation on the device's batches and on host copies of them: the same counts
    from types import SimpleNamespace
    from hiscache.hotness import embedding_cache_hit_rate
    table = torch.from_numpy(rng.standard_normal((len(batches), 4096)).astype(np.float32))

    def scores():
        it = iter(table)
        return lambda n, d: next(it)[:n].to(d)
    on_host = [SimpleNamespace(ptr=x.ptr.cpu(), idx=x.idx.cpu(), sub_to_full=x.sub_to_full.cpu(),
                               num_node_in_layer=x.num_node_in_layer) for x in batches]
    dev_run = list(embedding_cache_hit_rate(batches, N, rate=0.9, staleness=4, expire=True, score_fn=scores()))
    assert dev_run == list(embedding_cache_hit_rate(on_host, N, rate=0.9, staleness=4, expire=True, score_fn=scores()))
    assert dev_run[-1][0] > dev_run[0][0] and dev_run[-1][2][1] > 0


def test_embedding_cache_simulation_against_loops():
    """The simulation of /root/reference/test/test_cache.py:165-239 against its loops written out per row and per
    edge, with scores from a table both sides read; entries that expire, and (as there) entries that never do."""
    from types import SimpleNamespace
    from hiscache.hotness import embedding_cache_hit_rate
    rng = np.random.default_rng(5)
    N, L = 400, 3
    batches = []
    for _ in range(12):
        nnl = [10]
        for _k in range(L):
            nnl.append(nnl[-1] + int(rng.integers(5, 40)))
        deg = rng.integers(0, 5, size=nnl[L - 1])
        ptr = np.zeros(nnl[L - 1] + 1, np.int64)
        ptr[1:] = np.cumsum(deg)
        idx = np.zeros(ptr[-1], np.int64)
        for k in range(L):                       # a row of layer k draws its neighbours among layer k+1's nodes
            for r in range(nnl[k - 1] if k else 0, nnl[k]):
                idx[ptr[r]:ptr[r + 1]] = rng.integers(0, nnl[k + 1], size=deg[r])
        batches.append(SimpleNamespace(ptr=torch.from_numpy(ptr), idx=torch.from_numpy(idx),
                                       sub_to_full=torch.from_numpy(rng.choice(N, size=nnl[L], replace=False)),
                                       num_node_in_layer=torch.tensor(nnl)))
    scores = torch.from_numpy(rng.standard_normal((len(batches) * L + 1, 200)).astype(np.float32))

    def run_loops(cache_layers, staleness, expire):
        status = {k: np.zeros(N, np.int64) for k in cache_layers}
        admitted = {k: [] for k in cache_layers}
        out, draw = [], 0
        for it, b in enumerate(batches, start=1):
            nnl = b.num_node_in_layer.tolist()
            s2f, ptr, idx = b.sub_to_full.numpy(), b.ptr.numpy(), b.idx.numpy()
            useful = [np.ones(nnl[0], bool)]
            for k in range(L):
                nxt = np.zeros(nnl[k + 1], bool)
                for i in range(nnl[k]):
                    cached = k in status and status[k][s2f[i]] != 0
                    if useful[k][i] and not cached:
                        for e in range(ptr[i], ptr[i + 1]):
                            nxt[idx[e]] = True
                useful.append(nxt)
            hits = nnl[L] - int(useful[L].sum())
            for k in sorted(status):
                sc = scores[draw, :nnl[k]]
                draw += 1
                thres = float(torch.quantile(sc, 0.7))
                ids = [int(s2f[i]) for i in range(nnl[k]) if float(sc[i]) < thres and useful[k][i]]
                admitted[k].append(ids)
                for v in ids:
                    status[k][v] = it
                if it >= staleness:
                    for v in admitted[k].pop(0):
                        if expire and it - status[k][v] >= staleness:
                            status[k][v] = 0
            out.append((hits, nnl[L], {k: int((status[k] != 0).sum()) for k in sorted(status)}))
        return out

    for cache_layers, staleness, expire in (((1,), 4, True), ((1,), 4, False), ((1, 2), 3, True), ((0, 1, 2), 200, False)):
        draw = [0]

        def score_fn(n, device):
            draw[0] += 1
            return scores[draw[0] - 1, :n].to(device)
        got = list(embedding_cache_hit_rate(batches, N, cache_layers=cache_layers, rate=0.7, staleness=staleness,
                                            expire=expire, score_fn=score_fn))
        assert got == run_loops(cache_layers, staleness, expire), (cache_layers, staleness, expire)
    # without a cache only the rows that no edge reaches are spared; the caches spare more
    bare = list(embedding_cache_hit_rate(batches, N, cache_layers=()))
    assert sum(h for h, _, _ in got) > sum(h for h, _, _ in bare) and bare[0][2] == {}
    # the same batch twice with the seeds' layer cached: all seeds but the one with the largest score are held
    # (the quantile 1.0 is that score and admission is strict), so the second pass needs one seed's rows only
    twice = list(embedding_cache_hit_rate(batches[:1] * 2, N, cache_layers=(0,), rate=1.0,
                                          score_fn=lambda n, d: torch.arange(n, dtype=torch.float32)))
    assert twice[0][2] == {0: 9} and twice[1][0] > twice[0][0]
