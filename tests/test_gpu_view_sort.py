"""The transposed view of large blocks (more than 2^20 edge slots: the library's two-level bucket sort),
through the C ABI.

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


def stable_view(ptr, idx, R, N, E, hrow=None, hsrc=None):
    """(ptrT, order): the kept edge slots among the first E, sorted by source, slot order inside a source."""
    lim = min(int(ptr[R]), E)
    e = np.arange(int(ptr[0]), lim)
    row = np.searchsorted(ptr[1:R + 1], e, side="right")
    keep = (idx[e] >= 0) & (idx[e] < N)
    if hrow is not None:
        keep &= hrow[row] == -1
    if hsrc is not None:
        keep &= hsrc[np.clip(idx[e], 0, N - 1)] == -1
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


def _even_ptr(R, E):
    deg = np.full(R, E // R, np.int64)
    deg[: E - (E // R) * R] += 1
    ptr = np.zeros(R + 1, np.int64)
    np.cumsum(deg, out=ptr[1:])
    return ptr


def _adversarial_blocks():
    """(name, ptr, idx, N, row map, source map): blocks that put every edge into one bucket, leave none alive,
    end exactly on a tile, consist of one row, repeat one id across a wave, or have as many sources as the
    bucket sort takes (and one more, which goes to the library sort)."""
    rng = np.random.default_rng(17)
    R = 100_000
    E = 8192 * 129                                         # a whole number of tiles of 8 192 edge slots
    ptr = _even_ptr(R, E)
    ar = np.arange(E, dtype=np.int64)
    yield "one_source_takes_all", ptr, np.full(E, 7, np.int64), 1000, None, None
    yield "a_single_source", ptr, np.zeros(E, np.int64), 1, None, None
    yield "every_source_flagged", ptr, rng.integers(0, 50_000, size=E), 50_000, None, np.ones(50_000, np.int64)
    yield "every_row_flagged", ptr, rng.integers(0, 50_000, size=E), 50_000, np.ones(R, np.int64), None
    yield "one_row", np.array([0, E + 1], np.int64), rng.integers(0, 70_000, size=E + 1), 70_000, None, None
    yield "one_id_per_wave", ptr, (ar // 64) % 3_000_000, 3_000_000, None, None
    yield "two_ids_per_wave", ptr, (ar // 64) * 2 % 3_000_000 + (ar & 1), 3_000_000, None, None
    yield "two_far_ids", ptr, (ar & 1) * 2_999_999, 3_000_000, None, None
    yield "descending", ptr, 2_999_999 - (ar * 3_000_000) // E, 3_000_000, None, None
    for N in (5376 * 8192 - 1, 5376 * 8192 + 1):
        hs = np.where(rng.random(N) < 0.3, 1, -1).astype(np.int64)
        yield "most_sources_%d" % N, ptr, rng.integers(0, N, size=E), N, np.where(rng.random(R) < 0.2, 3, -1), hs


def test_bucket_sorted_view_on_adversarial_blocks(be):
    for name, ptr, idx, N, hrow, hsrc in _adversarial_blocks():
        R = len(ptr) - 1
        idx = np.ascontiguousarray(idx, np.int64)
        hrow = None if hrow is None else np.ascontiguousarray(hrow, np.int64)
        want_ptrT, order, rows = stable_view(ptr, idx, R, N, len(idx), hrow, hsrc)
        n = len(order)
        for want_edges in (False, True):
            ptrT, rowT, edgeT = be.build_transpose(T(ptr), T(idx), None if hrow is None else T(hrow), R, N,
                                                   want_edges=want_edges,
                                                   history_map_src=None if hsrc is None else T(hsrc))
            np.testing.assert_array_equal(ptrT.cpu().numpy(), want_ptrT, err_msg=name)
            np.testing.assert_array_equal(rowT.cpu().numpy()[:n], rows, err_msg=name)
            if want_edges:
                np.testing.assert_array_equal(edgeT.cpu().numpy()[:n], order, err_msg=name)
