"""The transposed view of large blocks (more than 2^20 edge slots: the library's two-level bucket sort)
and the per-edge substitution mask that the forward pass hands to it, through the C ABI.

Everything here is index work: bit-exact against NumPy's stable argsort (the definition of the view)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def T(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


@pytest.fixture(scope="module")
def be():
    import hiscache_backend
    hiscache_backend.load_library()
    assert torch.cuda.is_available()
    return hiscache_backend


def stable_view(ptr, idx, R, N, E, hrow=None, hsrc=None, drop=None):
    """(ptrT, order): the kept edge slots among the first E, sorted by source, slot order inside a source."""
    lim = min(int(ptr[R]), E)
    e = np.arange(int(ptr[0]), lim)
    row = np.searchsorted(ptr[1:R + 1], e, side="right")
    keep = (idx[e] >= 0) & (idx[e] < N)
    if hrow is not None:
        keep &= hrow[row] == -1
    if hsrc is not None:
        keep &= hsrc[np.clip(idx[e], 0, N - 1)] == -1
    if drop is not None:
        keep &= drop[e] == 0
    e, row = e[keep], row[keep]
    o = np.argsort(idx[e], kind="stable")
    ptrT = np.searchsorted(idx[e][o], np.arange(N + 1), side="left")
    return ptrT, e[o], row[o]


def ragged_block(rng, R, N, mean_deg, empty=0.0, hub_row=None, popular=None):
    deg = rng.poisson(mean_deg, size=R).astype(np.int64)
    if empty:
        deg[rng.random(R) < empty] = 0
    if hub_row is not None:
        deg[R // 2] = hub_row
    ptr = np.zeros(R + 1, np.int64)
    np.cumsum(deg, out=ptr[1:])
    idx = rng.integers(0, N, size=int(ptr[-1]), dtype=np.int64)
    if popular:
        idx[rng.random(len(idx)) < popular] = N // 3
    return ptr, idx


CASES = [
    # R, N, mean degree, share of empty rows, a hub row, share of edges onto one source
    (200_000, 1_500_000, 6.0, 0.0, None, None),     # every tile's rows are non-empty (bitmap row lookup)
    (350_000, 400_000, 5.0, 0.3, 40_000, None),     # empty rows in every tile (row search), a row across tiles
    (300_000, 60, 4.0, 0.0, None, None),            # fewer sources than buckets could hold: one source per bucket
    (150_000, 3_000_000, 8.0, 0.05, None, 0.2),     # a source with 240 k edges: its bucket is ranked from memory
    (1_200_000, 30_000_000, 2.0, 0.4, None, None),  # 13 local bits: many sources, few edges each
]


@pytest.mark.parametrize("R,N,deg,empty,hub_row,popular", CASES)
def test_bucket_sorted_view_is_the_stable_sort(be, R, N, deg, empty, hub_row, popular):
    rng = np.random.default_rng(R + N)
    ptr, idx = ragged_block(rng, R, N, deg, empty, hub_row, popular)
    E_all = len(idx)
    assert E_all > 1 << 20
    idx[rng.integers(0, E_all, size=20)] = N + 5          # ids outside the sources are left out
    idx[rng.integers(0, E_all, size=5)] = -3
    hrow = np.where(rng.random(R) < 0.2, 3, -1).astype(np.int64)
    hsrc = np.where(rng.random(N) < 0.3, 1, -1).astype(np.int64)
    hsrc[N // 3] = -1
    dptr, didx = T(ptr), T(idx)
    # all rows; a prefix of the rows over a prefix of the edge slots (a layer of a shared CSR)
    for Rl, E in ((R, E_all), (R * 2 // 3, int(ptr[R * 2 // 3]) + 777)):
        for use_row, use_src in ((False, False), (True, True)):
            want_ptrT, order, rows = stable_view(ptr, idx, Rl, N, E, hrow if use_row else None,
                                                 hsrc if use_src else None)
            n = len(order)
            for want_edges in (False, True):
                ptrT, rowT, edgeT = be.build_transpose(dptr, didx, T(hrow) if use_row else None, Rl, N,
                                                       num_edge=E, want_edges=want_edges,
                                                       history_map_src=T(hsrc) if use_src else None)
                np.testing.assert_array_equal(ptrT.cpu().numpy(), want_ptrT)
                np.testing.assert_array_equal(rowT.cpu().numpy()[:n], rows)
                if want_edges:
                    np.testing.assert_array_equal(edgeT.cpu().numpy()[:n], order)


def test_view_from_an_edge_mask_equals_the_view_from_the_source_map(be):
    """hc_build_transpose_edge_mask over what the forward pass noted per edge slot, on a small block (counting
    sort), a middle one (library sort) and a large one (bucket sort), with and without a row map."""
    for R, N, deg in ((3_000, 2_000, 6.0), (90_000, 30_000, 5.0), (260_000, 700_000, 5.0)):
        rng = np.random.default_rng(R)
        ptr, idx = ragged_block(rng, R, N, deg, 0.1)
        E = len(idx)
        hsrc = np.where(rng.random(N) < 0.4, 7, -1).astype(np.int64)
        hrow = np.where(rng.random(R) < 0.2, 3, -1).astype(np.int64)
        drop = (hsrc[idx] != -1).astype(np.uint8)
        for use_row in (False, True):
            hr = T(hrow) if use_row else None
            a = be.build_transpose(T(ptr), T(idx), hr, R, N, want_edges=True, history_map_src=T(hsrc))
            b = be.build_transpose(T(ptr), T(idx), hr, R, N, want_edges=True, edge_drop=T(drop))
            n = int(a[0][-1])
            assert torch.equal(a[0], b[0])
            assert torch.equal(a[1][:n], b[1][:n]) and torch.equal(a[2][:n], b[2][:n])
            want_ptrT, order, rows = stable_view(ptr, idx, R, N, E, hrow if use_row else None, None, drop)
            np.testing.assert_array_equal(b[0].cpu().numpy(), want_ptrT)
            np.testing.assert_array_equal(b[2].cpu().numpy()[:n], order)
    with pytest.raises(ValueError):
        be.build_transpose(T(ptr), T(idx), None, R, N, history_map_src=T(hsrc), edge_drop=T(drop))


@pytest.mark.parametrize("F", [256, 128, 100])
def test_forward_notes_the_substituted_edge_slots(be, F):
    """hc_aggr_fwd_src_mask: the same output as the plain launch, and edge_sub[e] = (hmap[idx[e]] != -1) for the
    edge slots of the first R rows (long rows and the generic width included); the autograd operator's backward,
    which builds its view from that mask, gives the gradient of the view built from the map."""
    rng = np.random.default_rng(F)
    R, N, Hn = 70_000, 50_000, 20_000
    ptr, idx = ragged_block(rng, R + 50, N, 6.0, 0.1, hub_row=3000)
    Rl = R
    feat = T(rng.standard_normal((N, F)).astype(np.float32))
    hist = T(rng.standard_normal((Hn, F)).astype(np.float32))
    hmap = np.where(rng.random(N) < 0.4, rng.integers(0, Hn, size=N), -1).astype(np.int64)
    dptr, didx, dmap = T(ptr), T(idx), T(hmap)
    plain = be._aggr_fwd(be.SUBST_SRC, dptr, didx, feat, dmap, hist, F, None, Rl)
    edge_sub = torch.full((len(idx),), 9, dtype=torch.uint8, device=DEV)
    noted = be._aggr_fwd(be.SUBST_SRC, dptr, didx, feat, dmap, hist, F, None, Rl, edge_sub=edge_sub)
    assert torch.equal(plain, noted)
    used = int(ptr[Rl])
    got = edge_sub.cpu().numpy()
    np.testing.assert_array_equal(got[:used], (hmap[idx[:used]] != -1).astype(np.uint8))
    assert (got[used:] == 9).all()                         # slots behind the first R rows are not touched
    # the operator: the gradient through the mask equals the gradient through the map
    x = feat.clone().requires_grad_(True)
    g = T(rng.standard_normal((Rl, F)).astype(np.float32))
    be.aggr_forward_source_history(x, dptr, didx, dmap, hist, num_node=Rl).backward(g)
    tr = be.build_transpose(dptr, didx, None, Rl, N, want_edges=False, history_map_src=dmap)
    want = be._aggr_bwd(dptr, didx, tr, g, None, None, feat, False, None, 0, Rl, N)[0]
    assert torch.equal(x.grad, want)
    assert (x.grad[dmap != -1] == 0).all()
