"""GPU parity of the aggregation kernels (forward, transpose, backward) against the CPU oracle,
through the C ABI (``hiscache_backend`` is a ctypes shim over ``libhiscache_hip.so``).

Bars: index outputs bit-exact; fp32 aggregates bit-exact against the oracle (same summation
order) and within 1e-5 relative of an fp64 closed form; fp16/bf16 inputs within 1e-2."""
import numpy as np
import pytest
import torch

from helpers import random_csr, random_hmap

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


CASES = [  # (R, N, F, maxdeg, hub, dtype)
    (300, 200, 256, 12, 300, torch.float32),   # fast path 16-byte loads, a row longer than one staging batch
    (300, 200, 128, 12, 130, torch.float32),   # 8-byte loads
    (257, 100, 64, 9, None, torch.float32),    # 4-byte loads
    (200, 150, 512, 20, 70, torch.float32),    # two chunks per lane
    (120, 90, 768, 6, None, torch.float32),    # three chunks
    (120, 90, 1024, 6, 65, torch.float32),     # four chunks
    (150, 120, 100, 10, 100, torch.float32),   # generic path (F not a multiple of 64)
    (90, 70, 172, 5, None, torch.float32),     # generic path
    (90, 70, 300, 5, None, torch.float32),     # generic path, more than one column tile
    (200, 150, 256, 12, 80, torch.float16),
    (200, 150, 768, 12, 80, torch.float16),    # mag240M-shaped rows
    (200, 150, 512, 12, None, torch.bfloat16),
    (64, 50, 1, 4, None, torch.float32),
]


@pytest.mark.parametrize("R,N,F,maxdeg,hub,dtype", CASES)
@pytest.mark.parametrize("with_hist", [False, True])
def test_fwd_mean_row_mode(be, orc, R, N, F, maxdeg, hub, dtype, with_hist):
    rng = np.random.default_rng(R * 7 + F)
    ptr, idx = random_csr(rng, R, N, maxdeg, hub=hub)
    x = T(rng.standard_normal((N, F)).astype(np.float32), dtype)
    x32 = x.float().cpu().numpy()
    if with_hist:
        hmap = random_hmap(rng, R, 0.35)
        hbuf = T(rng.standard_normal((R, F)).astype(np.float32), dtype)
        out = be.aggr_forward_history(x, T(ptr), T(idx), T(hmap), hbuf, F, R)
        ref = orc.fwd_mean_row(ptr, idx, x32, hmap, hbuf.float().cpu().numpy(), split_above=be.long_row_edges(F, dtype))
    else:
        out = be.aggr_forward_history(x, T(ptr), T(idx), none(), none(), 0, R)
        ref = orc.fwd_mean_row(ptr, idx, x32, None, None, split_above=be.long_row_edges(F, dtype))
    assert out.dtype == torch.float32 and out.requires_grad
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)


@pytest.mark.parametrize("R", [9000, 70000])
@pytest.mark.parametrize("mode", ["plain", "row", "src"])
def test_fwd_long_rows_quarter_rule(be, orc, mode, R):
    """Rows above the long-row threshold are summed as four quarters by a whole block: same bits as the
    oracle applying the documented quarter rule, and within 1e-5 of the strictly sequential sum.  With
    70000 rows the shim passes scratch and the long rows are listed and scheduled first."""
    rng = np.random.default_rng(42)
    N, F = 3000, 128
    ptr, idx = random_csr(rng, R, N, 6)
    deg = np.diff(ptr)
    for r in rng.choice(R, size=12, replace=False):           # a dozen long rows, one of them empty-adjacent
        deg[r] = int(rng.integers(257, 900))
    deg[R - 1] = 1500                                          # the very last row is long
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    idx = rng.integers(0, N, size=int(ptr[-1]), dtype=np.int64)
    x = rng.standard_normal((N, F)).astype(np.float32)
    if mode == "plain":
        out = be.aggr_forward_history(T(x), T(ptr), T(idx), none(), none(), 0, R)
        ref = orc.fwd_mean_row(ptr, idx, x, None, None, split_above=be.long_row_edges(F))
        seq = orc.fwd_mean_row(ptr, idx, x, None, None)
        assert (ref != seq).any()                              # the two orders really differ in rounding
        np.testing.assert_allclose(ref, seq, rtol=1e-5, atol=1e-6)
    elif mode == "row":
        hmap = random_hmap(rng, R, 0.4)
        hmap[R - 1] = -1
        hmap[np.flatnonzero(deg > 256)[:3]] = 7                # long rows that are history rows
        hbuf = rng.standard_normal((R, F)).astype(np.float32)
        out = be.aggr_forward_history(T(x), T(ptr), T(idx), T(hmap), T(hbuf), F, R)
        ref = orc.fwd_mean_row(ptr, idx, x, hmap, hbuf, split_above=be.long_row_edges(F))
    else:
        hist = rng.standard_normal((500, F)).astype(np.float32)
        hmap = np.where(rng.random(N) < 0.4, rng.integers(0, 500, size=N), -1).astype(np.int64)
        out = be.aggr_forward_source_history(T(x), T(ptr), T(idx), T(hmap), T(hist))
        ref = orc.fwd_mean_src(ptr, idx, x, hmap, hist, split_above=be.long_row_edges(F))
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)


def test_fwd_mean_closed_form_tolerance(be):
    """Against an fp64 closed form (independent of the oracle): 1e-5 relative."""
    rng = np.random.default_rng(1)
    R, N, F = 500, 400, 256
    ptr, idx = random_csr(rng, R, N, 40, hub=900)
    x = rng.standard_normal((N, F)).astype(np.float32)
    out = be.aggr_forward_history(T(x), T(ptr), T(idx), none(), none(), 0, 0).detach().cpu().numpy()
    deg = np.diff(ptr)
    ref = np.add.reduceat(x[idx].astype(np.float64), np.minimum(ptr[:-1], len(idx) - 1), axis=0)
    ref[deg == 0] = 0
    ref /= np.maximum(deg, 1)[:, None]
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-6)


def test_fwd_history_wider_than_features_and_num_node(be, orc):
    rng = np.random.default_rng(2)
    R, N, F, hs = 100, 80, 128, 160
    ptr, idx = random_csr(rng, R, N, 8)
    x = rng.standard_normal((N, F)).astype(np.float32)
    hmap = random_hmap(rng, R, 0.5)
    hbuf = rng.standard_normal((R, hs)).astype(np.float32)
    out = be.aggr_forward_history(T(x), T(ptr), T(idx), T(hmap), T(hbuf), hs, 61)
    ref = orc.fwd_mean_row(ptr, idx, x, hmap[:61], hbuf[:61], num_node=61)
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)
    # mixed dtypes: fp32 features, fp16 row-aligned history
    h16 = T(hbuf[:, :F]).half()
    out = be.aggr_forward_history(T(x), T(ptr), T(idx), T(hmap), h16, F, R)
    ref = orc.fwd_mean_row(ptr, idx, x, hmap, h16.float().cpu().numpy())
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)


@pytest.mark.parametrize("F,dtype", [(256, torch.float32), (128, torch.float32), (100, torch.float32),
                                     (256, torch.float16)])
def test_fwd_src_mode(be, orc, F, dtype):
    rng = np.random.default_rng(3)
    R, N, Hn = 400, 300, 120
    ptr, idx = random_csr(rng, R, N, 15, hub=200)
    feat = T(rng.standard_normal((N, F)).astype(np.float32), dtype)
    hist = T(0.5 * rng.standard_normal((Hn, F)).astype(np.float32), dtype)
    hmap = np.full(N, -1, np.int64)
    hit = rng.random(N) < 0.4
    hmap[hit] = rng.integers(0, Hn, size=int(hit.sum()))
    out = be.aggr_forward_source_history(feat, T(ptr), T(idx), T(hmap), hist)
    ref = orc.fwd_mean_src(ptr, idx, feat.float().cpu().numpy(), hmap, hist.float().cpu().numpy(),
                           split_above=be.long_row_edges(F, dtype))
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)
    # an all-miss map is the plain mean
    out2 = be.aggr_forward_source_history(feat, T(ptr), T(idx), T(np.full(N, -1, np.int64)), hist)
    out3 = be.aggr_forward_history(feat, T(ptr), T(idx), none(), none(), 0, 0)
    assert torch.equal(out2, out3)


@pytest.mark.parametrize("R,N,E_extra", [(200, 150, 0), (200, 150, 77), (1, 5, 0), (50, 3, 10)])
def test_build_transpose_bit_exact(be, orc, R, N, E_extra):
    rng = np.random.default_rng(4 + R)
    ptr, idx = random_csr(rng, R, N, 9, hub=150)
    idx_all = np.concatenate([idx, rng.integers(0, N, size=E_extra)]).astype(np.int64)  # edges of deeper layers
    hmap = random_hmap(rng, R, 0.3)
    for hm in (None, hmap):
        ptrT, rowT, edgeT = be.build_transpose(T(ptr), T(idx_all), None if hm is None else T(hm), R, N)
        rp, rr, re = orc.build_transpose(ptr, idx_all, hm, N, num_node=R)
        np.testing.assert_array_equal(ptrT.cpu().numpy(), rp)
        k = int(rp[-1])
        np.testing.assert_array_equal(rowT.cpu().numpy()[:k], rr)
        np.testing.assert_array_equal(edgeT.cpu().numpy()[:k], re)
        # the cheaper build without edge slots gives the same segments and rows
        ptrT2, rowT2, none_ = be.build_transpose(T(ptr), T(idx_all), None if hm is None else T(hm), R, N,
                                                 want_edges=False)
        assert none_ is None
        np.testing.assert_array_equal(ptrT2.cpu().numpy(), rp)
        np.testing.assert_array_equal(rowT2.cpu().numpy()[:k], rr)


def test_build_transpose_many_more_sources_than_edges(be, orc):
    rng = np.random.default_rng(9)
    R, N = 40, 5000                                   # sparse: the segment bounds come from a binary search
    ptr, idx = random_csr(rng, R, N, 5)
    for want in (True, False):
        ptrT, rowT, _ = be.build_transpose(T(ptr), T(idx), None, R, N, want_edges=want)
        rp, rr, _ = orc.build_transpose(ptr, idx, None, N)
        np.testing.assert_array_equal(ptrT.cpu().numpy(), rp)
        np.testing.assert_array_equal(rowT.cpu().numpy()[: int(rp[-1])], rr)


@pytest.mark.parametrize("R,N,deg,popular", [
    (3000, 40, 30, None),        # 90 k edges onto 40 sources: every segment is ranked through the LDS bitmap
    (20000, 5000, 12, 0.3),      # one source with ~70 k incoming edges beside short segments
    (4000, 900_000, 6, None),    # many sources without edges (still the counting-sort path)
    (262_144 // 4, 300, 4, None),  # exactly the largest block of the counting-sort path
    (70_000, 3000, 5, 0.2),      # above it: the library-sort path
    (5000, (1 << 20) + 5, 5, None),  # few edges but more sources than the counting sort takes
    (300_000, 50_000, 4, 0.1),   # 1.2 M edges: the library's radix passes (9-bit digits), 16-bit keys: two passes
    (270_000, 600_000, 4, None),  # the same with 20-bit keys: three passes
])
def test_build_transpose_paths_agree_with_a_stable_argsort(be, R, N, deg, popular):
    """The counting-sort path of small blocks and the library-sort path of large ones against NumPy's
    stable argsort: segment bounds, rows and edge slots, with long segments, dropped rows and dropped
    sources."""
    rng = np.random.default_rng(R + N)
    ptr = (np.arange(R + 1) * deg).astype(np.int64)
    idx = rng.integers(0, N, size=R * deg, dtype=np.int64)
    if popular:
        idx[rng.random(len(idx)) < popular] = N // 3
    hrow = random_hmap(rng, R, 0.2)
    hsrc = np.where(rng.random(N) < 0.3, 1, -1).astype(np.int64)
    hsrc[N // 3] = -1
    e = np.arange(len(idx))
    row = e // deg
    for use_row, use_src in ((False, False), (True, True)):
        keep = np.ones(len(idx), bool)
        if use_row:
            keep &= hrow[row] == -1
        if use_src:
            keep &= hsrc[idx] == -1
        order = e[keep][np.argsort(idx[keep], kind="stable")]
        want_ptrT = np.searchsorted(idx[order], np.arange(N + 1), side="left")
        for want_edges in (True, False):
            ptrT, rowT, edgeT = be.build_transpose(T(ptr), T(idx), T(hrow) if use_row else None, R, N,
                                                   want_edges=want_edges,
                                                   history_map_src=T(hsrc) if use_src else None)
            np.testing.assert_array_equal(ptrT.cpu().numpy(), want_ptrT)
            np.testing.assert_array_equal(rowT.cpu().numpy()[: len(order)], row[order])
            if want_edges:
                np.testing.assert_array_equal(edgeT.cpu().numpy()[: len(order)], order)


def test_build_transpose_no_edges(be):
    ptr = torch.zeros(11, dtype=torch.int64, device=DEV)
    idx = torch.zeros(0, dtype=torch.int64, device=DEV)
    ptrT, _, _ = be.build_transpose(ptr, idx, None, 10, 7)
    assert ptrT.cpu().tolist() == [0] * 8


@pytest.mark.parametrize("R,N,F,maxdeg,hub", [(300, 200, 256, 12, 300), (300, 250, 128, 12, 130),
                                               (200, 150, 64, 9, None), (150, 120, 512, 10, 70),
                                               (150, 120, 100, 10, 100), (90, 70, 300, 5, None)])
@pytest.mark.parametrize("with_hist", [False, True])
def test_bwd_mean_bit_exact_and_deterministic(be, orc, R, N, F, maxdeg, hub, with_hist):
    rng = np.random.default_rng(R + F)
    ptr, idx = random_csr(rng, R, N, maxdeg, hub=hub)
    x = T(rng.standard_normal((N, F)).astype(np.float32)).requires_grad_(True)
    g = rng.standard_normal((R, F)).astype(np.float32)
    if with_hist:
        hmap = random_hmap(rng, R, 0.35)
        hbuf = T(rng.standard_normal((R, F)).astype(np.float32)).requires_grad_(True)
        out = be.aggr_forward_history(x, T(ptr), T(idx), T(hmap), hbuf, F, R)
    else:
        hmap, hbuf = None, None
        out = be.aggr_forward_history(x, T(ptr), T(idx), none(), none(), 0, R)
    out.backward(T(g))
    gx, gh = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F), chunk=be.bwd_chunk_edges(F))
    np.testing.assert_array_equal(x.grad.cpu().numpy(), gx)
    if with_hist:
        np.testing.assert_array_equal(hbuf.grad.cpu().numpy(), gh)
    # run-to-run bit equality (no float atomics)
    first = x.grad.clone()
    x.grad = None
    out2 = be.aggr_forward_history(x, T(ptr), T(idx), none() if hmap is None else T(hmap),
                                   none() if hbuf is None else hbuf.detach(), 0 if hmap is None else F, R)
    out2.backward(T(g))
    assert torch.equal(first, x.grad)


@pytest.mark.parametrize("with_hist", [False, True])
def test_bwd_hub_sources_are_chunked(be, orc, with_hist):
    """Sources with more than 512 incoming edges (hubs of a sampled batch) are summed in chunks by
    independent waves: same bits as the oracle applying the documented chunk rule, 1e-5 from the
    strictly ordered sum.  Includes a hub at the first and at the last source id, hubs next to each
    other, sources without edges and a hub whose size is a multiple of the chunk."""
    rng = np.random.default_rng(77)
    R, N, F = 6000, 500, 128
    deg = rng.integers(0, 8, size=R)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    E = int(ptr[-1])
    idx = rng.integers(0, N, size=E, dtype=np.int64)
    hubs = {0: 1700, 1: 513, 2: 1024, 250: 3000, N - 1: 2200}
    pos = rng.permutation(E)
    o = 0
    for s_, k in hubs.items():
        idx[pos[o:o + k]] = s_
        o += k
    idx[idx == 7] = 8                                            # source 7 has no edges at all
    x = T(rng.standard_normal((N, F)).astype(np.float32)).requires_grad_(True)
    g = rng.standard_normal((R, F)).astype(np.float32)
    hmap = random_hmap(rng, R, 0.2) if with_hist else None
    if with_hist:
        hbuf = T(rng.standard_normal((R, F)).astype(np.float32)).requires_grad_(True)
        out = be.aggr_forward_history(x, T(ptr), T(idx), T(hmap), hbuf, F, R)
    else:
        out = be.aggr_forward_history(x, T(ptr), T(idx), none(), none(), 0, R)
    out.backward(T(g))
    C = be.bwd_chunk_edges(F)
    assert C == 512
    ref, _ = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F), chunk=C)
    seq, _ = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F))
    got = x.grad.cpu().numpy()
    np.testing.assert_array_equal(got, ref)
    assert (ref != seq).any()
    np.testing.assert_allclose(ref, seq, rtol=1e-4, atol=1e-5)
    assert (got[7] == 0).all()


def test_bwd_retain_grad_on_output_and_raw_feature_input(be, orc):
    """The op's output always requires grad so that the produced embedding can collect dL/d(out)
    even when the input is a raw feature tensor (history_aggr.cu:604)."""
    rng = np.random.default_rng(6)
    R, N, F = 60, 50, 128
    ptr, idx = random_csr(rng, R, N, 6)
    x = T(rng.standard_normal((N, F)).astype(np.float32))           # no grad
    out = be.aggr_forward_history(x, T(ptr), T(idx), none(), none(), 0, R)
    assert out.requires_grad
    out.retain_grad()
    w = T(rng.standard_normal((F, 3)).astype(np.float32)).requires_grad_(True)
    (out @ w).sum().backward()
    assert out.grad is not None and out.grad.shape == out.shape


@pytest.mark.parametrize("table_grad", [False, True])
def test_src_mode_backward(be, orc, table_grad):
    """Backward of the per-source substitution: a substituted source gets no gradient in ``feat`` (its
    row was not read); its share goes to the table's gradient when the table requires one."""
    rng = np.random.default_rng(7)
    R, N, F, Hn = 300, 200, 256, 150
    ptr, idx = random_csr(rng, R, N, 10, hub=90)
    feat = T(rng.standard_normal((N, F)).astype(np.float32)).requires_grad_(True)
    hist = T(rng.standard_normal((Hn, F)).astype(np.float32)).requires_grad_(table_grad)
    hmap = np.where(rng.random(N) < 0.4, rng.integers(0, Hn, size=N), -1).astype(np.int64)
    g = rng.standard_normal((R, F)).astype(np.float32)
    out = be.aggr_forward_source_history(feat, T(ptr), T(idx), T(hmap), hist)
    out.backward(T(g))
    gf, gh = orc.bwd_mean_src(ptr, idx, g, N, chunk=be.bwd_chunk_edges(F), hmap_src=hmap, hist_shape=(Hn, F))
    np.testing.assert_array_equal(feat.grad.cpu().numpy(), gf)
    assert (feat.grad.cpu().numpy()[hmap != -1] == 0).all()
    if table_grad:
        # rows shared by several sources are added by index_add_ (any order): compare with a tolerance
        np.testing.assert_allclose(hist.grad.cpu().numpy(), gh, rtol=1e-5, atol=1e-6)
    else:
        assert hist.grad is None


def test_transposed_view_drops_substituted_sources(be, orc):
    rng = np.random.default_rng(71)
    R, N = 500, 300
    ptr, idx = random_csr(rng, R + 20, N, 12, hub=200)
    hrow = random_hmap(rng, R, 0.3)
    hsrc = np.where(rng.random(N) < 0.4, 5, -1).astype(np.int64)
    ptrT, rowT, edgeT = be.build_transpose(T(ptr), T(idx), T(hrow), R, N, history_map_src=T(hsrc))
    e = np.arange(int(ptr[R]))
    row = np.searchsorted(ptr[1:R + 1], e, side="right")
    keep = (hrow[row] == -1) & (hsrc[idx[e]] == -1)
    order = e[keep][np.argsort(idx[e[keep]], kind="stable")]
    n = len(order)
    np.testing.assert_array_equal(edgeT.cpu().numpy()[:n], order)
    np.testing.assert_array_equal(rowT.cpu().numpy()[:n], row[order])
    want_ptrT = np.searchsorted(idx[order], np.arange(N + 1), side="left")
    np.testing.assert_array_equal(ptrT.cpu().numpy(), want_ptrT)


@pytest.mark.parametrize("table_dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("F,R", [(256, 300), (128, 300), (64, 70_000), (100, 200)])
def test_src_mode_table_narrower_than_features(be, orc, table_dtype, F, R):
    """Per-source substitution with fp32 features and an fp16 / bf16 table (the papers100M-shaped
    combination), fast widths and a generic width, long rows, a block above the long-row-list
    threshold: bit-exact against the checker on the table widened to fp32."""
    rng = np.random.default_rng(F + R)
    N, Hn = 5000, 3000
    ptr, idx = random_csr(rng, R, N, 12, hub=700)
    feat = rng.standard_normal((N, F)).astype(np.float32)
    hist = T(rng.standard_normal((Hn, F)).astype(np.float32)).to(table_dtype)
    hmap = np.where(rng.random(N) < 0.4, rng.integers(0, Hn, size=N), -1).astype(np.int64)
    out = be.aggr_forward_source_history(T(feat), T(ptr), T(idx), T(hmap), hist)
    ref = orc.fwd_mean_src(ptr, idx, feat, hmap, hist.float().cpu().numpy(), split_above=be.long_row_edges(F))
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)
    # narrower features than the table: refused
    with pytest.raises(ValueError):
        be.aggr_forward_source_history(T(feat).half(), T(ptr), T(idx), T(hmap), hist.float())


def test_src_mode_bitmap_over_many_sources(be, orc):
    """Above 2^20 sources the forward derives one bit per source from the map and consults it before
    the map: same bits out, with maps that are empty, full, and that end inside a 64-source group."""
    rng = np.random.default_rng(72)
    R, F = 3000, 64
    for N in ((1 << 20) + 37, (1 << 20) + 64):
        ptr, idx = random_csr(rng, R, N, 20, hub=900)
        idx[:50] = N - 1 - np.arange(50)              # the last sources, in the bitmap's last word
        feat = T(rng.standard_normal((N, F)).astype(np.float32))
        Hn = 1000
        hist = rng.standard_normal((Hn, F)).astype(np.float32)
        for frac in (0.4, 0.0, 1.0):
            hmap = np.where(rng.random(N) < frac, rng.integers(0, Hn, size=N), -1).astype(np.int64)
            out = be.aggr_forward_source_history(feat, T(ptr), T(idx), T(hmap), T(hist))
            ref = orc.fwd_mean_src(ptr, idx, feat.cpu().numpy(), hmap, hist, split_above=be.long_row_edges(F))
            np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)


@pytest.mark.parametrize("F,H", [(64, 1), (256, 1), (96, 1), (32, 3), (256, 2),
                                 # several heads on the fast widths: heads of 8, 16, 32 lanes and of 2 chunks
                                 (32, 8), (64, 4), (128, 2), (512, 2), (64, 3)])
@pytest.mark.parametrize("hist_kind", ["none", "shared", "concat"])
def test_edge_value_variants(be, orc, F, H, hist_kind):
    rng = np.random.default_rng(F + H)
    R, N = 120, 90
    ptr, idx = random_csr(rng, R, N, 8, hub=700)     # one row above the long-row threshold (never split with heads)
    E = len(idx)
    multi = H > 1
    vin = rng.standard_normal((N, H, F) if multi else (N, F)).astype(np.float32)
    ev = rng.standard_normal((E, H) if multi else (E,)).astype(np.float32)
    g = rng.standard_normal((R, H, F) if multi else (R, F)).astype(np.float32)
    if hist_kind == "none":
        hmap, hbuf, hs = None, None, 0
    else:
        hs = F * H if (hist_kind == "concat" and multi) else F
        hmap = random_hmap(rng, R, 0.3)
        hbuf = rng.standard_normal((R, hs)).astype(np.float32)
    x = T(vin).requires_grad_(True)
    evt = T(ev).requires_grad_(True)
    hb = None if hbuf is None else T(hbuf).requires_grad_(True)
    out = be.aggr_forward_history_edge_value(x, T(ptr), T(idx), evt, none() if hmap is None else T(hmap),
                                             none() if hb is None else hb, hs, R)
    # single-head weighted sums on the fast widths follow the quarter rule for long rows
    ref = orc.fwd_edge_value(ptr, idx, ev, vin, hmap, hbuf, split_above=0 if multi else be.long_row_edges(F))
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)
    out.backward(T(g))
    gx, gh, eg = orc.bwd_edge_value(ptr, idx, ev, g, hmap, vin, N, hsize=hs, want_edge_grad=True)
    np.testing.assert_array_equal(x.grad.cpu().numpy(), gx)
    if hb is not None:
        np.testing.assert_array_equal(hb.grad.cpu().numpy(), gh)
    # edge_grad: dot products, summation order differs from the oracle's fp64 -> tolerance scaled by sum |terms|
    deg = np.diff(ptr)
    dst = np.repeat(np.arange(R), deg)
    scale = (np.abs(g[dst]) * np.abs(vin[idx])).sum(-1)
    err = np.abs(evt.grad.cpu().numpy() - eg)
    assert (err <= 1e-5 * scale + 1e-7).all()


def test_empty_inputs(be):
    ptr = torch.zeros(1, dtype=torch.int64, device=DEV)
    idx = torch.zeros(0, dtype=torch.int64, device=DEV)
    x = torch.zeros((5, 128), device=DEV)
    out = be.aggr_forward_history(x, ptr, idx, none(), none(), 0, 0)
    assert out.shape == (0, 128)
    # rows without any edge
    ptr = torch.zeros(9, dtype=torch.int64, device=DEV)
    out = be.aggr_forward_history(x, ptr, idx, none(), none(), 0, 8)
    assert out.shape == (8, 128) and (out == 0).all()
    out.sum().backward()


def test_shim_rejects_bad_arguments(be):
    x = torch.zeros((4, 128), device=DEV)
    ptr = torch.zeros(5, dtype=torch.int64, device=DEV)
    idx = torch.zeros(0, dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError):
        be.aggr_forward_history(x, ptr.int(), idx, none(), none(), 0, 4)        # wrong index dtype
    with pytest.raises(ValueError):
        be.aggr_forward_history(x, ptr, idx, none(), none(), 0, 9)              # more rows than ptr has
    with pytest.raises(ValueError):
        be.aggr_forward_history(x.double(), ptr, idx, none(), none(), 0, 4)     # unsupported dtype
    with pytest.raises(ValueError):
        be.aggr_forward_history(x.t(), ptr, idx, none(), none(), 0, 4)          # not contiguous
    with pytest.raises(ValueError):
        be.aggr_forward_history(x, ptr, idx, torch.full((2,), -1, device=DEV), x, 128, 4)  # short map


def test_fwd_long_row_list_overflow_falls_back(be, orc):
    """Scratch that cannot hold every long row: the list is ignored and the rows are summed in place,
    with the same bits."""
    import ctypes
    rng = np.random.default_rng(43)
    R, N, F = 70000, 2000, 64
    ptr, idx = random_csr(rng, R, N, 4)
    deg = np.diff(ptr)
    deg[rng.choice(R, size=9, replace=False)] = 300
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    idx = rng.integers(0, N, size=int(ptr[-1]), dtype=np.int64)
    x = rng.standard_normal((N, F)).astype(np.float32)
    ref = orc.fwd_mean_row(ptr, idx, x, None, None, split_above=be.long_row_edges(F))
    lib = be.load_library()
    tp, ti, tx = T(ptr), T(idx), T(x)
    for ws_ints in (4, 64):                                    # room for 4 rows (overflow) and for 64
        out = torch.full((R, F), float("nan"), device=DEV)
        ws = torch.empty(256 + 4 * ws_ints, dtype=torch.uint8, device=DEV)
        rc = lib.hc_aggr_fwd(0, tp.data_ptr(), ti.data_ptr(), tx.data_ptr(), 0, None, None, 0, 0, None, 1,
                             out.data_ptr(), R, F, N, ws.data_ptr(), ws.numel(),
                             torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        np.testing.assert_array_equal(out.cpu().numpy(), ref)


def test_check_csr_reports_bad_blocks(be):
    rng = np.random.default_rng(44)
    R, N = 500, 300
    ptr, idx = random_csr(rng, R, N, 7)
    be.check_csr(T(ptr), T(idx), R, N)                          # a valid block passes
    bad_idx = idx.copy(); bad_idx[[3, 10]] = [N, -1]
    with pytest.raises(ValueError, match="2 neighbour ids"):
        be.check_csr(T(ptr), T(bad_idx), R, N)
    bad_ptr = ptr.copy(); bad_ptr[100] = bad_ptr[101] + 5       # row 99 overshoots, row 100 runs backwards
    with pytest.raises(ValueError, match="1 rows end before"):
        be.check_csr(T(bad_ptr), T(idx), R, N)
    long_ptr = ptr.copy(); long_ptr[-1] += 4                    # the last row reaches past idx
    with pytest.raises(ValueError, match="offsets outside"):
        be.check_csr(T(long_ptr), T(idx), R, N)
    # ids behind ptr[R] are nobody's business
    tail = np.concatenate([idx, np.array([10**9], np.int64)])
    be.check_csr(T(ptr), T(tail), R, N)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_weighted_fast_path_prefix_rows_and_dtypes(be, orc, dtype):
    """Single-head weighted aggregation on a fast width over a row prefix: edge slots behind the last
    used row get a zero edge gradient, history rows too; fp16 inputs accumulate in fp32."""
    rng = np.random.default_rng(46)
    R_all, R, N, F = 500, 380, 300, 128
    ptr, idx = random_csr(rng, R_all, N, 9, hub=900)
    E = len(idx)
    vin = T(rng.standard_normal((N, F)).astype(np.float32), dtype)
    v32 = vin.float().cpu().numpy()
    ev = rng.standard_normal(E).astype(np.float32)
    g = rng.standard_normal((R, F)).astype(np.float32)
    hmap = random_hmap(rng, R, 0.3)
    hbuf = rng.standard_normal((R, F)).astype(np.float32)
    x = vin.clone().requires_grad_(True)
    evt = T(ev).requires_grad_(True)
    out = be.aggr_forward_history_edge_value(x, T(ptr), T(idx), evt, T(hmap), T(hbuf), F, R)
    ref = orc.fwd_edge_value(ptr[: R + 1], idx, ev, v32, hmap, hbuf, split_above=be.long_row_edges(F, dtype))
    np.testing.assert_array_equal(out.detach().cpu().numpy(), ref)
    out.backward(T(g))
    gx, _, eg = orc.bwd_edge_value(ptr[: R + 1], idx, ev, g, hmap, v32, N, hsize=F, want_edge_grad=True)
    got_gx = x.grad.float().cpu().numpy()
    if dtype == torch.float32:
        np.testing.assert_array_equal(got_gx, gx)
    else:
        np.testing.assert_allclose(got_gx, gx, rtol=1e-2, atol=1e-2 * np.abs(gx).max())
    got = evt.grad.cpu().numpy()
    used = int(ptr[R])
    assert (got[used:] == 0).all() and used < E
    dst = np.repeat(np.arange(R), np.diff(ptr[: R + 1]))
    hist_edge = hmap[dst] != -1
    assert (got[:used][hist_edge] == 0).all() and hist_edge.any()
    scale = (np.abs(g[dst]) * np.abs(v32[idx[:used]])).sum(-1)
    assert (np.abs(got[:used] - eg[:used]) <= 1e-5 * scale + 1e-7).all()


def test_c_abi_from_a_program_without_python():
    """tests/abi_demo/abi_demo (built against the library): hipMalloc'd buffers, raw pointers, status
    codes; it checks forward, transposed view and backward of a 4-row block against hand-worked values."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "abi_demo", "abi_demo")
    assert os.path.exists(exe), "abi_demo is built by make -C tests/abi_demo"
    p = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0 and p.stdout.startswith("abi_demo: ok"), (p.returncode, p.stdout, p.stderr)
