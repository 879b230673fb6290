"""Seeded random shapes through the aggregation entry points, bit for bit against the CPU checker:
row counts on both sides of the large-block threshold (long-row list, XCD block order), skewed
degrees with several long rows and hub sources, all history fractions, fast and generic widths."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def be():
    import hiscache_backend
    hiscache_backend.load_library()
    return hiscache_backend


def T(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def skewed_block(rng, R, N, mean_deg, n_long, n_hub_src):
    deg = np.minimum(rng.zipf(1.8, size=R), 60) * rng.integers(0, 2, size=R)       # many empty rows
    deg = (deg * mean_deg / max(deg.mean(), 1e-9)).astype(np.int64)
    if n_long:
        deg[rng.choice(R, size=n_long, replace=False)] = rng.integers(257, 1400, size=n_long)
    ptr = np.zeros(R + 1, np.int64)
    np.cumsum(deg, out=ptr[1:])
    E = int(ptr[-1])
    idx = rng.integers(0, N, size=E, dtype=np.int64)
    for s in rng.choice(N, size=n_hub_src, replace=False):                          # popular sources
        idx[rng.random(E) < min(0.5, 900 / max(E, 1))] = s
    return ptr, idx


CASES = [  # (seed, R, N, F, mean_deg, n_long, n_hub_src, hist_frac)
    (1, 0, 10, 64, 3, 0, 0, 0.0),
    (2, 1, 1, 256, 3, 0, 0, 1.0),
    (3, 4097, 900, 128, 4, 3, 1, 0.3),
    (4, 65535, 5000, 64, 3, 5, 2, 0.5),
    (5, 65536, 5000, 64, 3, 5, 2, 0.0),
    (6, 65537, 3000, 128, 2, 9, 0, 1.0),
    (7, 131072 + 5, 7000, 64, 2, 12, 3, 0.4),
    (8, 70001, 4000, 100, 2, 4, 1, 0.4),              # generic width: no list, no quarter rule
    (9, 2048 * 9 + 1, 777, 192, 5, 6, 2, 0.2),
    (10, 300, 100000, 64, 6, 2, 0, 0.3),              # many more sources than edges
    (11, 200_000, 9000, 256, 2, 20, 2, 0.3),          # well above the large-block threshold, widest fast loads
    (12, 262_144, 20000, 128, 2, 7, 1, 0.0),
]


@pytest.mark.parametrize("seed,R,N,F,mean_deg,n_long,n_hub_src,hist_frac", CASES)
def test_random_block_forward_backward(be, orc, seed, R, N, F, mean_deg, n_long, n_hub_src, hist_frac):
    rng = np.random.default_rng(1000 + seed)
    ptr, idx = skewed_block(rng, R, N, mean_deg, min(n_long, R), min(n_hub_src, N)) if R else (np.zeros(1, np.int64), np.zeros(0, np.int64))
    print("random case", seed, "R", R, "E", len(idx), "N", N, "F", F, flush=True)
    x = rng.standard_normal((N, F)).astype(np.float32)
    g = rng.standard_normal((R, F)).astype(np.float32)
    hmap = np.where(rng.random(R) < hist_frac, np.arange(R), -1).astype(np.int64) if hist_frac > 0 else None
    hbuf = rng.standard_normal((R, F)).astype(np.float32) if hmap is not None else None
    xt = T(x).requires_grad_(True)
    none = torch.empty(0, device=DEV)
    if R == 0:
        out = be.aggr_forward_history(xt, T(ptr), T(idx), none, none, 0, 0)
        assert out.shape == (0, F)
        return
    if hmap is not None:
        ht = T(hbuf).requires_grad_(True)
        out = be.aggr_forward_history(xt, T(ptr), T(idx), T(hmap), ht, F, R)
    else:
        out = be.aggr_forward_history(xt, T(ptr), T(idx), none, none, 0, R)
    ref = orc.fwd_mean_row(ptr, idx, x, hmap, hbuf, split_above=be.long_row_edges(F))
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)
    out.backward(T(g))
    gx, gh = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F), chunk=be.bwd_chunk_edges(F))
    np.testing.assert_array_equal(xt.grad.cpu().numpy(), gx)
    if hmap is not None:
        np.testing.assert_array_equal(ht.grad.cpu().numpy(), gh)
    # the same gradient over a view of the whole block with nothing left out (history rows stepped over
    # in the kernel), for the first two thirds of the rows as well
    view = be.build_batch_view(T(ptr), T(idx), R, N)
    for Rl in (R, (2 * R) // 3):
        hm_l = None if hmap is None else hmap[:Rl]
        gv, ghv = be._aggr_bwd_batch_view(T(ptr), view, T(g[:Rl]), None if hm_l is None else T(hm_l), (Rl, F), F,
                                          Rl, N, want_hist_grad=hmap is not None)
        wv, whv = orc.bwd_mean_row_batch_view(ptr, idx, g[:Rl], hm_l, N, R, hbuf_shape=(Rl, F),
                                              chunk=be.bwd_chunk_edges(F))
        np.testing.assert_array_equal(gv.cpu().numpy(), wv)
        if hmap is not None:
            np.testing.assert_array_equal(ghv.cpu().numpy(), whv)
    # transposed view with edge slots, against the stable-sort statement
    ptrT, rowT, edgeT = be.build_transpose(T(ptr), T(idx), None if hmap is None else T(hmap), R, N)
    wp, wr, we = orc.build_transpose(ptr, idx, hmap, N)
    np.testing.assert_array_equal(ptrT.cpu().numpy(), wp)
    np.testing.assert_array_equal(rowT.cpu().numpy()[: len(wr)], wr)
    np.testing.assert_array_equal(edgeT.cpu().numpy()[: len(we)], we)
    # per-source substitution over the same block
    hist = rng.standard_normal((64, F)).astype(np.float32)
    smap = np.where(rng.random(N) < 0.4, rng.integers(0, 64, size=N), -1).astype(np.int64)
    out_s = be.aggr_forward_source_history(T(x), T(ptr), T(idx), T(smap), T(hist))
    np.testing.assert_array_equal(out_s.cpu().numpy(),
                                  orc.fwd_mean_src(ptr, idx, x, smap, hist, split_above=be.long_row_edges(F)))
    # single-head weighted sums over the same block (fast widths take the gather kernels too)
    ev = rng.standard_normal(len(idx)).astype(np.float32)
    xw = T(x).requires_grad_(True)
    evt = T(ev).requires_grad_(True)
    if hmap is not None:
        out_w = be.aggr_forward_history_edge_value(xw, T(ptr), T(idx), evt, T(hmap), T(hbuf), F, R)
    else:
        out_w = be.aggr_forward_history_edge_value(xw, T(ptr), T(idx), evt, none, none, 0, R)
    np.testing.assert_array_equal(out_w.detach().cpu().numpy(),
                                  orc.fwd_edge_value(ptr, idx, ev, x, hmap, hbuf, split_above=be.long_row_edges(F)))
    out_w.backward(T(g))
    gxw, _, egw = orc.bwd_edge_value(ptr, idx, ev, g, hmap, x, N, hsize=F, want_edge_grad=True)
    np.testing.assert_array_equal(xw.grad.cpu().numpy(), gxw)
    dst = np.repeat(np.arange(R), np.diff(ptr))
    scale = (np.abs(g[dst]) * np.abs(x[idx])).sum(-1)
    assert (np.abs(evt.grad.cpu().numpy() - egw) <= 1e-5 * scale + 1e-7).all()

