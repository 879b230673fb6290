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
        # (a view that knows it holds no hub: the backward then runs without its hub launches)
        known = be.BatchView(view.ptrT, view.rowT, view.edgeT, view.rows, view.n_src, view.num_edge,
                             max_in_degree=int(np.bincount(idx).max()))
        got = []
        for v in (None, view, known):
            xx = T(x).requires_grad_(True)
            hb = hbuf.clone().requires_grad_(True)
            out = be.aggr_forward_history(xx, tptr, tidx, hmap, hb, F, R, int(ptr[R]), v)
            out.backward(g)
            got.append((out.detach(), xx.grad, hb.grad))
        for a, b, c in zip(*got):
            assert torch.equal(a, b) and torch.equal(a, c)
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


def _stable_view(ptr, idx, R, n_src):
    """NumPy statement of the view: edges of the first R rows in stable order of their source."""
    E = int(ptr[R])
    dst = np.repeat(np.arange(R), np.diff(ptr[:R + 1]))
    order = np.argsort(idx[:E], kind="stable")
    ptrT = np.zeros(n_src + 1, np.int64)
    np.cumsum(np.bincount(idx[:E], minlength=n_src), out=ptrT[1:])
    return ptrT, dst[order].astype(np.int32), order.astype(np.int32)


@pytest.mark.parametrize("R,n_src,max_deg,hub_edges,slack", [
    (3000, 2000, 9, 700, 0),             # one window of edge slots, capacities equal to the sizes
    (9000, 3000, 12, 3000, 5000),        # capacities above the sizes
    (120000, 50000, 9, 9000, 200000),    # more than 2^18 edge slots: hubs ranked over several windows
    (10, 2000, 0, 0, 100),               # no edge at all
])
def test_view_with_sizes_on_the_device(be, R, n_src, max_deg, hub_edges, slack):
    """hc_build_transpose_dev reads R, E and n_src from device memory (launches sized by capacities):
    the same view as a stable NumPy sort, with and without edge slots."""
    rng = np.random.default_rng(R + n_src)
    deg = rng.integers(0, max_deg + 1, size=R)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    E = int(ptr[-1])
    idx = rng.integers(0, n_src, size=E, dtype=np.int64)
    if hub_edges:
        pos = rng.permutation(E)
        idx[pos[:hub_edges]] = 5                        # a hub whose slots are spread over the whole block
        idx[pos[hub_edges:hub_edges + 65]] = n_src - 1   # just above a wave's worth
        idx[pos[hub_edges + 65:hub_edges + 129]] = 0     # exactly a wave's worth
    max_E, max_src = E + slack, n_src + (slack // 7)
    idx_cap = np.concatenate([idx, np.full(max_E - E, -7, np.int64)])     # capacity beyond the block: never read
    sizes = T(np.array([R, E, n_src], np.int64))
    want_ptrT, want_rowT, want_edgeT = _stable_view(ptr, idx, R, n_src)
    flag = torch.full((1,), 7, dtype=torch.int32, device=DEV)
    longest = torch.full((2,), -5, dtype=torch.int64, device=DEV)
    for want_edges in (False, True):
        ptrT, rowT, edgeT = be.build_transpose_dev(T(ptr), T(idx_cap), sizes[0:1], sizes[1:2], sizes[2:3], max_E,
                                                   max_src, want_edges=want_edges, overflow=flag,
                                                   max_in_degree=longest[:1] if want_edges else None)
        # the largest in-degree, on request (one word: the next one stays as it was)
        assert longest.tolist() == ([int(np.bincount(idx, minlength=1).max()) if E else 0, -5] if want_edges
                                    else [-5, -5])
        np.testing.assert_array_equal(ptrT[: n_src + 1].cpu().numpy(), want_ptrT)
        np.testing.assert_array_equal(rowT[:E].cpu().numpy(), want_rowT)
        if want_edges:
            np.testing.assert_array_equal(edgeT[:E].cpu().numpy(), want_edgeT)
        assert int(flag) == 0


def test_view_with_sizes_beyond_the_capacities_is_flagged(be):
    """Sizes on the device that exceed what the launch was sized for are clamped (nothing is accessed out of
    bounds) and the overflow word says so: the view is then that of the truncated block."""
    rng = np.random.default_rng(5)
    R, n_src, deg = 400, 300, 5
    ptr = (np.arange(R + 1) * deg).astype(np.int64)
    idx = rng.integers(0, n_src, size=R * deg, dtype=np.int64)
    E = R * deg
    flag = torch.zeros(1, dtype=torch.int32, device=DEV)
    cut = 1200                                              # capacity for 1200 of the 2000 edge slots
    sizes = T(np.array([R, E, n_src], np.int64))
    ptrT, rowT, _ = be.build_transpose_dev(T(ptr), T(idx), sizes[0:1], sizes[1:2], sizes[2:3], cut, n_src,
                                           overflow=flag)
    assert int(flag) == 1
    want_ptrT, want_rowT, _ = _stable_view(ptr[: cut // deg + 1], idx[:cut], cut // deg, n_src)
    np.testing.assert_array_equal(ptrT.cpu().numpy(), want_ptrT)
    np.testing.assert_array_equal(rowT[:cut].cpu().numpy(), want_rowT)
    for bad in ([R, E, n_src + 50], [-1, E, n_src], [R, -3, n_src]):
        flag.zero_()
        be.build_transpose_dev(T(ptr), T(idx), *[T(np.array([v], np.int64)) for v in bad], E, n_src, overflow=flag)
        assert int(flag) == 1, bad
    be.build_transpose_dev(T(ptr), T(idx), sizes[0:1], sizes[1:2], sizes[2:3], E, n_src, overflow=flag)
    assert int(flag) == 0


@pytest.mark.parametrize("fanout,n_seed", [([5, 3], 64), ([15, 10, 5], 1200)])
def test_sampler_emits_the_view_with_the_batch(be, orc, fanout, n_seed):
    """NeighborSampler(emit_view=True): batch.view is the stable transposed view of batch.ptr / batch.idx,
    for consecutive batches, also when sampled ahead on the sampler's stream; the batch itself is the one
    the plain sampler draws."""
    from helpers import power_law_graph
    from hiscache import NeighborSampler
    rng = np.random.default_rng(31 + n_seed)
    n = 60000
    indptr, indices = power_law_graph(rng, n, 6.0, max_degree=3000)
    plain = NeighborSampler(indptr, indices, fanout, seed=4, device=DEV)
    emitting = NeighborSampler(indptr, indices, fanout, seed=4, device=DEV, emit_view=True)
    pending = None
    for it in range(3):
        seeds = torch.from_numpy(rng.choice(n, size=n_seed, replace=False).astype(np.int64)).to(DEV)
        print("view case", fanout, n_seed, it, flush=True)
        a = plain.sample(seeds)
        b = emitting.sample_async(seeds).get() if it else emitting.sample(seeds)
        assert torch.equal(a.ptr, b.ptr) and torch.equal(a.idx, b.idx) and torch.equal(a.sub_to_full, b.sub_to_full)
        L = len(fanout)
        R, n_all = int(b.num_node_in_layer[L - 1]), int(b.num_node_in_layer[L])
        v = b.view
        assert (v.rows, v.n_src, v.num_edge) == (R, n_all, b.idx.numel())
        assert v.max_in_degree == int(torch.bincount(b.idx).max())     # read back with the batch's sizes
        want_ptrT, want_rowT, _ = _stable_view(b.ptr.cpu().numpy(), b.idx.cpu().numpy(), R, n_all)
        np.testing.assert_array_equal(v.ptrT.cpu().numpy(), want_ptrT)
        np.testing.assert_array_equal(v.rowT[: v.num_edge].cpu().numpy(), want_rowT)
        o_ptrT, o_rowT, _ = orc.build_transpose(b.ptr.cpu().numpy(), b.idx.cpu().numpy(), None, n_all, R)
        np.testing.assert_array_equal(want_ptrT, o_ptrT)
        np.testing.assert_array_equal(want_rowT, o_rowT)
    assert int((emitting.node_map != 0x7fffffff).sum()) == 0
    del pending


@pytest.mark.parametrize("F,K,with_mask", [(256, 5, True), (64, 3, False), (768, 2, True), (128, 1, False)])
def test_relational_backward_over_the_batch_view_bit_exact(be, orc, F, K, with_mask):
    """hc_aggr_bwd_batch_view_typed against the oracle: relations outside [0, K), a relation array shorter
    than the edge list, sources ruled out by the used mask, a layer that owns a prefix of the view's rows,
    a source with hundreds of edges."""
    rng = np.random.default_rng(F + K)
    rows, sources = [400, 3000], [3000, 5000]
    ptr, idx = layered_csr(rng, rows, sources, 8, hubs={3: 700, 2999: 150})
    R_all, n_all = rows[-1], sources[-1]
    tptr, tidx = T(ptr), T(idx)
    view = be.build_batch_view(tptr, tidx, R_all, n_all, want_edges=True)
    for R, n_src in zip(rows, sources):
        rel = rng.integers(-1, K + 1, size=int(ptr[R]) - 3).astype(np.int64)
        used = (rng.random(n_src) < 0.8) if with_mask else None
        g = rng.standard_normal((R * K, F)).astype(np.float32)
        got = be._aggr_bwd_typed_batch_view(tptr, view, T(rel), K, None if used is None else T(used), T(g), R, n_src)
        want = orc.bwd_typed_batch_view(ptr[:R + 1], idx, rel, K, g, n_src, used)
        np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_relational_layer_with_and_without_the_batch_view(be):
    """The fused relational layer gives the same bits whether backward reads the batch's view or builds the
    view of its regrouped block (relations that follow from the edge's ends)."""
    from hiscache.history_model import MyRGCNConvHistory2
    rng = np.random.default_rng(8)
    torch.manual_seed(8)
    rows, sources = [300, 2500], [2500, 4000]
    ptr, idx = layered_csr(rng, rows, sources, 9, hubs={1: 600})
    K, Fin, H = 4, 256, 128
    tptr, tidx = T(ptr), T(idx)
    view = be.build_batch_view(tptr, tidx, rows[-1], sources[-1], want_edges=True)
    conv = MyRGCNConvHistory2(Fin, H, K, need_grad=True).to(DEV)
    R, n_src = rows[0], sources[0]
    et = T(((idx * 5 + 1) % K)[: int(ptr[R])])
    used = T(rng.random(n_src) < 0.85)
    hmap = T(random_hmap(rng, R, 0.3))
    hbuf = T(rng.standard_normal((R, H)).astype(np.float32))
    x0 = rng.standard_normal((n_src, Fin)).astype(np.float32)
    g = T(rng.standard_normal((R, H)).astype(np.float32))
    res = []
    for v in (None, view):
        x = T(x0).requires_grad_(True)
        conv.zero_grad()
        out, _ = conv(x, tptr, tidx, et, None, hmap, hbuf, used, H, R, view=v)
        out.backward(g)
        res.append((out.detach(), x.grad, conv.linear.grad.clone()))
    for a, b in zip(*res):
        assert torch.equal(a, b)
    assert float(res[1][1].abs().max()) > 0
