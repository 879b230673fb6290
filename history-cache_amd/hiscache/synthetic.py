"""Seeded synthetic inputs: graphs, layered-CSR mini-batches and kernel microbenchmark blocks.

The mini-batch layout is the one the reference's model and cache consume
(/root/reference/hiscache/history_model.py:120-153, history_cache.py:307-324): sub-graph nodes are
numbered seeds first, then every deeper hop's new nodes; ``num_node_in_layer[k]`` is the number of
nodes within k hops (so ``[0]`` = seeds, ``[-1]`` = all); one shared CSR (``ptr``, ``idx``) holds
the sampled neighbours of the first ``num_node_in_layer[L-1]`` nodes, and conv i uses its first
``num_node_in_layer[L-1-i]`` rows.
"""
from types import SimpleNamespace

import numpy as np
import torch


def uniform_graph(num_nodes, avg_degree, seed):
    """CSR of a directed graph with Poisson(avg_degree) out-degrees and uniform targets."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(avg_degree, size=num_nodes).astype(np.int64)
    indptr = np.zeros(num_nodes + 1, np.int64)
    np.cumsum(deg, out=indptr[1:])
    indices = rng.integers(0, num_nodes, size=int(indptr[-1]), dtype=np.int64)
    return indptr, indices


def zipf_degrees(n_rows, total_edges, alpha, max_degree, rng):
    """Power-law degrees in [1, max_degree] that sum to exactly ``total_edges``."""
    deg = np.minimum(rng.zipf(alpha, size=n_rows), max_degree).astype(np.float64)
    deg = np.maximum(1, np.minimum(max_degree, np.floor(deg * (total_edges / deg.sum())))).astype(np.int64)
    diff = int(total_edges - deg.sum())
    # spread the remainder one edge at a time over random rows that have room
    while diff != 0:
        step = 1 if diff > 0 else -1
        room = np.flatnonzero(deg < max_degree) if step > 0 else np.flatnonzero(deg > 1)
        pick = rng.choice(room, size=min(abs(diff), room.size), replace=False)
        deg[pick] += step
        diff -= step * pick.size
    return deg


def power_law_block(n_rows, total_edges, n_src, alpha=2.1, max_degree=5000, seed=2, device="cpu",
                    source_alpha=None):
    """One CSR block for the aggregation microbenchmark: ``n_rows`` destination rows with power-law
    degrees summing to ``total_edges`` and source ids over ``n_src`` nodes (uniform, or Zipf-popular
    when ``source_alpha`` is given).  Returns int64 torch tensors (ptr, idx)."""
    rng = np.random.default_rng(seed)
    deg = zipf_degrees(n_rows, total_edges, alpha, max_degree, rng)
    ptr = np.zeros(n_rows + 1, np.int64)
    np.cumsum(deg, out=ptr[1:])
    if source_alpha is None:
        idx = rng.integers(0, n_src, size=total_edges, dtype=np.int64)
    else:
        idx = (rng.zipf(source_alpha, size=total_edges) - 1) % n_src
        idx = (idx * 2654435761 % n_src).astype(np.int64)  # scatter the popular ids over the range
    return torch.from_numpy(ptr).to(device), torch.from_numpy(idx).to(device)


def sample_layered_batch(indptr, indices, seeds, fanout, rng):
    """Neighbour sampling without replacement, one sample per node, shared by all layers.

    ``fanout[k]`` neighbours are drawn for nodes first reached at hop k.  Returns a dict with
    ptr, idx, sub_to_full, num_node_in_layer (all NumPy int64)."""
    seeds = np.asarray(seeds, np.int64)
    sub_to_full = list(seeds.tolist())
    local = {int(v): i for i, v in enumerate(sub_to_full)}
    ptr = [0]
    idx = []
    num_node_in_layer = [len(sub_to_full)]
    frontier = (0, len(sub_to_full))
    for f in fanout:
        for u in range(frontier[0], frontier[1]):
            full = sub_to_full[u]
            nb = indices[indptr[full]:indptr[full + 1]]
            if nb.size > f:
                nb = rng.choice(nb, size=f, replace=False)
            for v in nb.tolist():
                j = local.get(v)
                if j is None:
                    j = len(sub_to_full)
                    local[v] = j
                    sub_to_full.append(v)
                idx.append(j)
            ptr.append(len(idx))
        frontier = (frontier[1], len(sub_to_full))
        num_node_in_layer.append(len(sub_to_full))
    return {
        "ptr": np.asarray(ptr, np.int64),
        "idx": np.asarray(idx, np.int64),
        "sub_to_full": np.asarray(sub_to_full, np.int64),
        "num_node_in_layer": np.asarray(num_node_in_layer, np.int64),
    }


def make_batch(sample, labels, device, emit_view=False, view_edges=False):
    """Wrap a sampled sub-graph as the batch object the cache and the model read.  ``emit_view``: the
    batch also carries the transposed view of its CSR (``batch.view``), as a loader that prepares
    batches ahead of the training step emits it (``NeighborSampler(emit_view=True)`` does); ``view_edges``
    adds the view's edge slots (read by the relational layer's backward)."""
    batch = _make_batch(sample, labels, device)
    if emit_view and torch.device(device).type == "cuda":
        import hiscache_backend
        L = len(sample["num_node_in_layer"]) - 1
        nnl = sample["num_node_in_layer"]
        batch.view = hiscache_backend.build_batch_view(batch.ptr, batch.idx, int(nnl[L - 1]), int(nnl[L]),
                                                       want_edges=view_edges)
        # known here at no cost (the arrays are on the host): lets the backward leave its hub path out
        idx = sample["idx"]
        batch.view.max_in_degree = int(np.bincount(idx, minlength=1).max()) if len(idx) else 0
    return batch


def _make_batch(sample, labels, device):
    n_seed = int(sample["num_node_in_layer"][0])
    L = len(sample["num_node_in_layer"]) - 1
    ptr = sample["ptr"]
    nnl = sample["num_node_in_layer"]
    num_edge_in_layer = [int(ptr[nnl[k]]) for k in range(L)]
    return SimpleNamespace(
        ptr=torch.from_numpy(sample["ptr"]).to(device),
        idx=torch.from_numpy(sample["idx"]).to(device),
        sub_to_full=torch.from_numpy(sample["sub_to_full"]).to(device),
        num_node_in_layer=torch.from_numpy(sample["num_node_in_layer"]),  # stays on the host
        num_edge_in_layer=num_edge_in_layer,
        y=torch.as_tensor(labels[sample["sub_to_full"][:n_seed]]).to(device),
        x=None,
        edge_type=None,
        typed_num_node_in_layer=None,
        view=None,
    )


def direct_power_law_batch(total_num_node, n_seed, fanout, alpha, seed, popularity_alpha=None,
                           degree_scale=1.0):
    """A sampled batch drawn directly (no full graph is materialised): every node reached at hop k
    gets min(max(1, floor(Zipf(alpha) * degree_scale)), fanout[k]) neighbours whose full ids are
    uniform (or Zipf-popular) over ``total_num_node``.  For graphs too large to build on the host
    (hundreds of millions of nodes); ``degree_scale`` sets the mean degree of the underlying graph."""
    rng = np.random.default_rng(seed)
    seeds = rng.choice(total_num_node, size=n_seed, replace=False).astype(np.int64)
    sub_to_full = seeds.copy()
    num_node_in_layer = [n_seed]
    ptr_parts = [np.zeros(1, np.int64)]
    idx_parts = []
    lo, hi = 0, n_seed
    n_edges = 0
    for f in fanout:
        n_front = hi - lo
        raw = np.minimum(rng.zipf(alpha, size=n_front), 1 << 20).astype(np.float64)
        deg = np.minimum(np.maximum(1, np.floor(raw * degree_scale)), f).astype(np.int64)
        e = int(deg.sum())
        if popularity_alpha is None:
            nb_full = rng.integers(0, total_num_node, size=e, dtype=np.int64)
        else:
            nb_full = ((rng.zipf(popularity_alpha, size=e) - 1) * 2654435761 % total_num_node).astype(np.int64)
        # local ids: existing nodes keep theirs, new ones are appended in first-seen order
        allv = np.concatenate([sub_to_full, nb_full])
        uniq, first = np.unique(allv, return_index=True)
        order = np.argsort(first, kind="stable")
        rank = np.empty_like(order)
        rank[order] = np.arange(order.size)
        loc = rank[np.searchsorted(uniq, nb_full)]
        new_full = uniq[order][sub_to_full.size:]
        sub_to_full = np.concatenate([sub_to_full, new_full])
        idx_parts.append(loc.astype(np.int64))
        ptr_parts.append(n_edges + np.cumsum(deg))
        n_edges += e
        lo, hi = hi, sub_to_full.size
        num_node_in_layer.append(sub_to_full.size)
    return {
        "ptr": np.concatenate(ptr_parts).astype(np.int64),
        "idx": np.concatenate(idx_parts).astype(np.int64) if idx_parts else np.zeros(0, np.int64),
        "sub_to_full": sub_to_full.astype(np.int64),
        "num_node_in_layer": np.asarray(num_node_in_layer, np.int64),
    }


def lognormal_grads(n_rows, width, mu=-3.0, sigma=1.5, seed=4, device="cpu", generator=None):
    """Gradient rows with random directions and LogNormal(mu, sigma) L2 norms (fp32)."""
    g = generator or torch.Generator(device=device).manual_seed(seed)
    d = torch.randn(n_rows, width, device=device, generator=g)
    d /= d.norm(dim=1, keepdim=True)
    norms = torch.exp(mu + sigma * torch.randn(n_rows, device=device, generator=g))
    d *= norms[:, None]
    return d


def batched_history_layer(samples, target_edges):
    """The history layer of many sampled batches side by side as one CSR block: for every batch its first
    num_node_in_layer[1] rows (the 1-hop nodes) with their edges, source ids shifted so that the batches'
    num_node_in_layer[2] sources do not overlap.  ``samples`` (results of direct_power_law_batch or of the
    sampler) are repeated until the block holds ``target_edges`` edges.  Returns (ptr, idx, rows, edges,
    sources) with numpy int64 arrays."""
    rows, cols, e_tot, k = 0, 0, 0, 0
    ptrs, idxs = [np.zeros(1, np.int64)], []
    while e_tot < target_edges:
        smp = samples[k % len(samples)]
        n1, n2 = int(smp["num_node_in_layer"][1]), int(smp["num_node_in_layer"][2])
        p = smp["ptr"][: n1 + 1]
        e = int(p[-1])
        ptrs.append(p[1:] + e_tot)
        idxs.append(smp["idx"][:e] + cols)
        e_tot += e
        rows += n1
        cols += n2
        k += 1
    return np.concatenate(ptrs), np.concatenate(idxs), rows, e_tot, cols

