"""The mini-batch's shared transposed view: one view of the whole batch CSR, emitted with the batch,
serves the backward of every layer (``hc_aggr_bwd_batch_view``), so that no view is built inside
backward.  Bars: bit-exact against the oracle's statement of the same summation order; the same bits
as the per-layer path wherever no source has more than a chunk of edges in the batch view."""
import numpy as np
import pytest
import torch

from helpers import random_hmap

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def T(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    return t.to(dtype) if dtype is not None else t


def none():
    return torch.empty(0, device=DEV)


@pytest.fixture(scope="module")
def be():
    import hiscache_backend
    hiscache_backend.load_library()
    assert torch.cuda.is_available()
    return hiscache_backend


def layered_csr(rng, rows, sources, max_deg, hubs=None):
    """A CSR whose first rows[k] rows only reach the first sources[k] nodes (k ascending = layers from
    the seeds outwards), as a sampled batch does.  ``hubs``: {source: edges} planted in the whole block."""
    R_all = rows[-1]
    deg = rng.integers(0, max_deg + 1, size=R_all)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    dst = np.repeat(np.arange(R_all), deg)
    bound = np.empty(R_all, np.int64)
    lo = 0
    for r, n in zip(rows, sources):
        bound[lo:r] = n
        lo = r
    idx = (rng.random(len(dst)) * bound[dst]).astype(np.int64)
    if hubs:
        pos = rng.permutation(len(dst))
        o = 0
        for s_, k in hubs.items():
            sel = pos[o:o + k]
            idx[sel] = s_
            o += k
    assert (idx < bound[dst]).all()
    return ptr, idx


@pytest.mark.parametrize("F", [256, 128, 64, 768, 100])
@pytest.mark.parametrize("with_hist", [False, True])
def test_batch_view_backward_bit_exact(be, orc, F, with_hist):
    """Three layers over one view, hubs at the first source, in the middle and next to each other."""
    rng = np.random.default_rng(F + (1 if with_hist else 0))
    rows, sources = [300, 2500, 9000], [2500, 9000, 12000]
    hubs = {0: 1700, 1: 513, 2: 1024, 40: 600, 2499: 900}
    ptr, idx = layered_csr(rng, rows, sources, 7, hubs)
    R_all, n_all = rows[-1], sources[-1]
    tptr, tidx = T(ptr), T(idx)
    view = be.build_batch_view(tptr, tidx, R_all, n_all)
    C = be.bwd_chunk_edges(F)
    for R, n_src in zip(rows, sources):
        g = rng.standard_normal((R, F)).astype(np.float32)
        hmap = random_hmap(rng, R, 0.3) if with_hist else None
        gx, gh = be._aggr_bwd_batch_view(tptr, view, T(g), None if hmap is None else T(hmap), (R, F), F, R,
                                         n_src, want_hist_grad=with_hist)
        ref, ref_h = orc.bwd_mean_row_batch_view(ptr, idx, g, hmap, n_src, R_all, hbuf_shape=(R, F), chunk=C)
        np.testing.assert_array_equal(gx.cpu().numpy(), ref)
        if with_hist:
            np.testing.assert_array_equal(gh.cpu().numpy(), ref_h)
        seq, _ = orc.bwd_mean_row(ptr[:R + 1], idx, g, hmap, n_src, hbuf_shape=(R, F))
        np.testing.assert_allclose(ref, seq, rtol=1e-3, atol=1e-4)   # sums of up to 1 700 terms
        if C and R == R_all:
            assert (ref != seq).any()                     # the hubs' chunk order is visible in the bits


@pytest.mark.parametrize("F", [256, 128, 100])
def test_batch_view_equals_layer_view_without_hubs(be, orc, F):
    """No source with more than a chunk of edges in the batch view: the same bits as the operator that
    builds a view per layer, through autograd, for every layer and with a history map."""
    rng = np.random.default_rng(5 + F)
    rows, sources = [200, 1500, 6000], [1500, 6000, 9000]
    ptr, idx = layered_csr(rng, rows, sources, 6)
    assert np.bincount(idx).max() <= 512
    tptr, tidx = T(ptr), T(idx)
    view = be.build_batch_view(tptr, tidx, rows[-1], sources[-1])
    for R, n_src in zip(rows, sources):
        x = rng.standard_normal((n_src, F)).astype(np.float32)
        g = T(rng.standard_normal((R, F)).astype(np.float32))
        hmap = T(random_hmap(rng, R, 0.35))
        hbuf = T(rng.standard_normal((R, F)).astype(np.float32))
        got = []
        for v in (None, view):
            xx = T(x).requires_grad_(True)
            hb = hbuf.clone().requires_grad_(True)
            out = be.aggr_forward_history(xx, tptr, tidx, hmap, hb, F, R, int(ptr[R]), v)
            out.backward(g)
            got.append((out.detach(), xx.grad, hb.grad))
        for a, b in zip(*got):
            assert torch.equal(a, b)
        ref, ref_h = orc.bwd_mean_row(ptr[:R + 1], idx, g.cpu().numpy(), hmap.cpu().numpy(), n_src,
                                      hbuf_shape=(R, F))
        np.testing.assert_array_equal(got[1][1].cpu().numpy(), ref)
        np.testing.assert_array_equal(got[1][2].cpu().numpy(), ref_h)


def test_batch_view_rejects_a_layer_it_does_not_cover(be):
    rng = np.random.default_rng(3)
    ptr, idx = layered_csr(rng, [50, 200], [200, 400], 4)
    view = be.build_batch_view(T(ptr), T(idx), 50, 200, num_edge=int(ptr[50]))
    g = torch.zeros(200, 64, device=DEV)
    with pytest.raises(ValueError):
        be._aggr_bwd_batch_view(T(ptr), view, g, None, None, 0, 200, 400)
