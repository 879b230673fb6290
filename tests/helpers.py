"""Shared generators for the tests (small seeded CSR blocks and cache states)."""
import numpy as np


def random_csr(rng, n_rows, n_src, max_deg, zero_frac=0.2, hub=None):
    """CSR with degrees in [0, max_deg]; a fraction of rows is empty; optional hub row degree."""
    deg = rng.integers(1, max_deg + 1, size=n_rows)
    deg[rng.random(n_rows) < zero_frac] = 0
    if hub is not None and n_rows > 0:
        deg[rng.integers(0, n_rows)] = hub
    ptr = np.zeros(n_rows + 1, np.int64)
    np.cumsum(deg, out=ptr[1:])
    idx = rng.integers(0, n_src, size=int(ptr[-1]), dtype=np.int64)
    return ptr, idx


def random_hmap(rng, n, frac):
    h = np.full(n, -1, np.int64)
    hit = rng.random(n) < frac
    h[hit] = rng.integers(0, 1000, size=int(hit.sum()))
    return h


def layered_batch(rng, n_full, n_seed, fanout, avg_deg=8):
    """A small layered-CSR mini-batch (see hiscache.synthetic.sample_layered_batch)."""
    from hiscache.synthetic import sample_layered_batch, uniform_graph
    indptr, indices = uniform_graph(n_full, avg_deg, int(rng.integers(1 << 30)))
    seeds = rng.choice(n_full, size=n_seed, replace=False)
    return sample_layered_batch(indptr, indices, seeds, fanout, rng)


def power_law_graph(rng, num_nodes, degree_scale, alpha=2.0, max_degree=2000, popular=True):
    """CSR of a directed graph with Zipf(alpha) out-degrees (scaled, capped) and neighbour ids skewed
    towards popular nodes (a cubed uniform scattered by a multiplicative hash), multi-edges possible:
    the shape of a citation graph, small enough to hold on the host."""
    raw = np.minimum(rng.zipf(alpha, size=num_nodes), 1 << 20).astype(np.float64)
    deg = np.minimum(np.floor(raw * degree_scale), max_degree).astype(np.int64)
    indptr = np.zeros(num_nodes + 1, np.int64)
    np.cumsum(deg, out=indptr[1:])
    E = int(indptr[-1])
    if popular:
        u = rng.random(E)
        indices = ((u * u * u * num_nodes).astype(np.int64) * 2654435761) % num_nodes
    else:
        indices = rng.integers(0, num_nodes, size=E, dtype=np.int64)
    return indptr, indices.astype(np.int64)
