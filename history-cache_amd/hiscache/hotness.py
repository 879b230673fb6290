"""Hotness orders: which nodes' feature rows are worth keeping in device memory.

The feature cache of ``HistoryCache`` and the hot tier of ``PinnedFeatureStore`` take the head of
``processed/sorted_indices.dat`` (node ids, hottest LAST; /root/reference/hiscache/history_cache.py:124-134).  The
reference ranks nodes by one of three metrics, spelled out in /root/reference/test/test_cache.py: the degree
(:18-24), how often a node turns up in the sampled batches of an epoch (:27-38), or a PageRank seeded at the
training nodes (:41-77); ``get_cache_map`` (:128-143) takes the top of the ranking and ``test_cache`` (:146-161)
measures the share of a batch's rows it serves; ``test_embedding_cache`` (:165-239) simulates embedding caches and
counts the input rows they spare.  The same functions here, on torch tensors (any device).
"""
import os
from os import path

import numpy as np
import torch


def degree_metric(indptr):
    """Number of adjacency entries of every node (test_cache.py:18-24)."""
    indptr = torch.as_tensor(indptr)
    return indptr[1:] - indptr[:-1]


def profile_metric(sampler, seeds, batch_size, num_epochs=1, generator=None):
    """How often every node appears in the batches that ``sampler`` (a ``NeighborSampler``) draws for ``seeds``
    in ``num_epochs`` shuffled passes (test_cache.py:27-38)."""
    seeds = torch.as_tensor(seeds).to(sampler.device)
    metric = torch.zeros(sampler.num_nodes, dtype=torch.int64, device=sampler.device)
    for _ in range(num_epochs):
        order = seeds[torch.randperm(seeds.numel(), device=seeds.device, generator=generator)]
        for lo in range(0, order.numel(), batch_size):
            batch = sampler.sample(order[lo:lo + batch_size].contiguous())
            metric[batch.sub_to_full] += 1            # a batch holds a node once
    return metric


def pagerank_metric(indptr, indices, train_idx, num_iter, damping=0.95):
    """PageRank over the undirected CSR with the mass started at the training nodes (test_cache.py:41-77):
    ``score <- (1 - d)/N + d * (score/deg + A (score/deg))`` for ``num_iter`` rounds."""
    indptr, indices = torch.as_tensor(indptr), torch.as_tensor(indices)
    n = indptr.numel() - 1
    train_idx = torch.as_tensor(train_idx).to(indptr.device)
    score = torch.full((n,), 1.0 / n, dtype=torch.float32, device=indptr.device)
    score[train_idx] = (n / train_idx.numel()) / n
    deg = (indptr[1:] - indptr[:-1]).clamp(min=1).to(torch.float32)
    lengths = indptr[1:] - indptr[:-1]
    for _ in range(int(num_iter)):
        score = score / deg
        score = score + torch.segment_reduce(score[indices], "sum", lengths=lengths, unsafe=True)
        score = (1.0 - damping) / n + damping * score
    return score


def hotness_order(metric):
    """Node ids by ascending metric, ties by ascending id: the hottest node LAST, as ``sorted_indices.dat`` holds
    them."""
    metric = torch.as_tensor(metric)
    return torch.sort(metric, stable=True).indices.to(torch.int64)


def get_cache_map(metric, cache_num):
    """Boolean mask of the nodes whose metric reaches that of the ``cache_num``-th hottest node
    (test_cache.py:128-143; ties at the threshold are all taken, as there)."""
    metric = torch.as_tensor(metric)
    if cache_num <= 0:
        return torch.zeros_like(metric, dtype=torch.bool)
    if cache_num >= metric.numel():
        return torch.ones_like(metric, dtype=torch.bool)
    ranked = torch.sort(metric, descending=True, stable=True).indices
    return metric >= metric[ranked[cache_num]]


def feature_cache_hit_rate(cache_status, batches):
    """Share of the batches' nodes whose features the cached set holds (test_cache.py:146-161).
    Returns (rate, hits, visits)."""
    visits = hits = 0
    for batch in batches:
        nodes = batch.sub_to_full
        visits += int(nodes.numel())
        hits += int(cache_status[nodes].sum())
    return (hits / visits if visits else 0.0), hits, visits


def embedding_cache_hit_rate(batches, num_nodes, cache_layers=(1,), rate=0.9, staleness=200, expire=False,
                             score_fn=None):
    """Simulate embedding caches on a stream of batches and count the input rows they spare
    (test_cache.py:165-239).  Layer k's cache holds nodes whose layer-k embedding is stored (k = 0: the seeds).
    Per batch, top down: a layer-k row must be computed when it is needed and not cached; the neighbours of such
    rows are needed in layer k+1 (:165-175, :201-208); an input row that is not needed is a hit (:211-213).
    Then every layer of ``cache_layers`` admits its needed rows whose score lies under the ``rate`` quantile of
    the layer's scores (:215-225; ``score_fn(n, device)``, default standard normal as there).
    ``expire``: drop the entries admitted ``staleness`` iterations ago.  The reference writes that reset into a
    temporary (:226-230), so its entries never expire: False reproduces it, True does what it means to.
    Yields (hits, visits, entries held per layer) after every batch."""
    status = {k: None for k in cache_layers}
    admitted = {k: [] for k in cache_layers}
    glb_iter = 0
    for batch in batches:
        glb_iter += 1
        s2f, ptr, idx = batch.sub_to_full, batch.ptr, batch.idx
        dev = s2f.device
        nnl = [int(n) for n in batch.num_node_in_layer]
        L = len(nnl) - 1
        for k in status:
            if status[k] is None:
                status[k] = torch.zeros(int(num_nodes), dtype=torch.int64, device=dev)
        needed = [torch.ones(nnl[0], dtype=torch.bool, device=dev)]
        for k in range(L):
            live = needed[k]
            if k in status:
                live = live & (status[k][s2f[:nnl[k]]] == 0)
            deg = ptr[1:nnl[k] + 1] - ptr[:nnl[k]]
            nxt = torch.zeros(nnl[k + 1], dtype=torch.bool, device=dev)
            nxt[idx[:int(ptr[nnl[k]])][torch.repeat_interleave(live, deg)]] = True
            needed.append(nxt)
        visits = nnl[L]
        hits = visits - int(needed[L].sum())
        for k in sorted(status):
            if k >= L:
                continue
            score = (score_fn or (lambda n, d: torch.randn(n, device=d)))(nnl[k], dev)
            thres = torch.quantile(score, rate)
            to_cache = s2f[:nnl[k]][(score < thres) & needed[k]]
            admitted[k].append(to_cache)
            status[k][to_cache] = glb_iter
            if glb_iter >= staleness:
                oldest = admitted[k].pop(0)
                if expire:
                    stale = oldest[glb_iter - status[k][oldest] >= staleness]
                    status[k][stale] = 0
        yield hits, visits, {k: int((status[k] != 0).sum()) for k in sorted(status)}


def write_hotness_order(root, order):
    """Write ``order`` (hottest last) as ``<root>/processed/sorted_indices.dat``."""
    d = path.join(str(root), "processed")
    os.makedirs(d, exist_ok=True)
    np.ascontiguousarray(torch.as_tensor(order).cpu().numpy(), dtype=np.int64).tofile(path.join(d, "sorted_indices.dat"))
    return path.join(d, "sorted_indices.dat")
