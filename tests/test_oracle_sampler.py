"""The sequential statement of the layered sampler, pinned by what its rule implies (no reference
sampler exists: the reference takes batches from an external loader)."""
import numpy as np
import pytest


def simple_graph(rng, n, max_deg, hubs=0):
    """CSR without multi-edges: every node gets a random subset of the others."""
    deg = rng.integers(0, max_deg + 1, size=n)
    if hubs:
        deg[rng.choice(n, size=hubs, replace=False)] = min(n - 1, 40 * max_deg)
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(deg, out=indptr[1:])
    indices = np.concatenate([rng.choice(n, size=d, replace=False) for d in deg]).astype(np.int64)
    return indptr, indices


def test_perm_is_a_bijection(orc):
    for d in list(range(2, 130)) + [255, 256, 257, 1000, 4097]:
        for key in (0, 1, 0xDEADBEEFCAFEF00D):
            img = sorted(orc.sample_perm(j, d, key) for j in range(d))
            assert img == list(range(d)), (d, key)


def test_perm_depends_on_key(orc):
    a = [orc.sample_perm(j, 1000, 5) for j in range(50)]
    b = [orc.sample_perm(j, 1000, 6) for j in range(50)]
    assert a != b


def check_batch(b, indptr, indices, seeds, fanout):
    L = len(fanout)
    nnl, ptr, idx, s2f = b["num_node_in_layer"], b["ptr"], b["idx"], b["sub_to_full"]
    assert nnl[0] == len(seeds) and (s2f[: len(seeds)] == seeds).all()
    assert len(np.unique(s2f)) == len(s2f) == nnl[L]
    assert len(ptr) == nnl[L - 1] + 1 and ptr[0] == 0 and ptr[-1] == len(idx) == b["num_edge_in_layer"][-1]
    for k in range(L):
        assert b["num_edge_in_layer"][k] == ptr[nnl[k]]
    # rows: min(d, fanout) picks, all from the node's list, distinct (the graph has no multi-edges)
    bounds = [0] + list(nnl)
    for k in range(L):
        for u in range(bounds[k], bounds[k + 1]):
            f = s2f[u]
            adj = indices[indptr[f]:indptr[f + 1]]
            got = s2f[idx[ptr[u]:ptr[u + 1]]]
            assert len(got) == min(len(adj), fanout[k])
            if len(adj) <= fanout[k]:
                assert (got == adj).all()
            else:
                assert len(set(got.tolist())) == len(got) and set(got.tolist()) <= set(adj.tolist())
    # local ids are handed out in first-seen order
    new = [v for v in dict.fromkeys(idx.tolist()) if v >= len(seeds)]
    assert new == list(range(len(seeds), max(new, default=len(seeds) - 1) + 1))
    # a node first reached at hop k+1 is numbered in [nnl[k], nnl[k+1])
    for k in range(L):
        rows = idx[ptr[bounds[k]]:ptr[bounds[k + 1]]]
        assert rows.max(initial=-1) < nnl[k + 1]


@pytest.mark.parametrize("fanout", [[4], [5, 3], [6, 4, 2]])
def test_sample_layers_structure(orc, fanout):
    rng = np.random.default_rng(100 + len(fanout))
    indptr, indices = simple_graph(rng, 400, 9, hubs=3)
    seeds = rng.choice(400, size=30, replace=False).astype(np.int64)
    b = orc.sample_layers(indptr, indices, seeds, fanout, 1234)
    check_batch(b, indptr, indices, seeds, fanout)
    again = orc.sample_layers(indptr, indices, seeds, fanout, 1234)
    other = orc.sample_layers(indptr, indices, seeds, fanout, 1235)
    assert all((b[k] == again[k]).all() for k in b)
    assert not np.array_equal(other["sub_to_full"], b["sub_to_full"])


def test_sample_positions_are_uniform(orc):
    """One node of degree 20, fanout 5, 4000 different keys: every list position is picked about
    equally often (chi-square with 19 degrees of freedom; 60 is far beyond the 0.9999 quantile)."""
    d, f, runs = 20, 5, 4000
    indptr = np.array([0, d] + [d] * d, np.int64)            # node 0 points at nodes 1..d
    indices = np.arange(1, d + 1, dtype=np.int64)
    hits = np.zeros(d + 1)
    pairs = np.zeros((d + 1, d + 1))
    for s in range(runs):
        b = orc.sample_layers(indptr, indices, np.array([0]), [f], s)
        picked = b["sub_to_full"][b["idx"]]
        assert len(set(picked.tolist())) == f
        hits[picked] += 1
        pairs[np.ix_(picked, picked)] += 1
    expect = runs * f / d
    chi2 = ((hits[1:] - expect) ** 2 / expect).sum()
    assert chi2 < 60, chi2
    # pairs of positions too: each unordered pair has probability f(f-1)/(d(d-1))
    iu = np.triu_indices(d, 1)
    pe = runs * f * (f - 1) / (d * (d - 1))
    chi2p = ((pairs[1:, 1:][iu] - pe) ** 2 / pe).sum()
    assert chi2p < 190 + 6 * np.sqrt(2 * 189), chi2p
