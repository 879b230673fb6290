"""Pins the CPU oracle's aggregation routines against closed forms (SciPy CSR products, SDDMM),
brute force on tiny graphs and invariants.  No GPU."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from helpers import random_csr, random_hmap


def brute_fwd_mean(ptr, idx, vin, hmap, hbuf):
    R, F = len(ptr) - 1, vin.shape[1]
    out = np.zeros((R, F), np.float64)
    for r in range(R):
        if hmap is not None and hmap[r] != -1:
            out[r] = hbuf[r, :F]
            continue
        nb = idx[ptr[r]:ptr[r + 1]]
        if len(nb):
            out[r] = vin[nb].astype(np.float64).sum(0) / len(nb)
    return out


@pytest.mark.parametrize("seed,R,N,F,maxdeg", [(0, 40, 30, 7, 5), (1, 50, 50, 64, 9), (2, 10, 5, 130, 70)])
def test_fwd_mean_brute_and_scipy(orc, seed, R, N, F, maxdeg):
    rng = np.random.default_rng(seed)
    ptr, idx = random_csr(rng, R, N, maxdeg)
    vin = rng.standard_normal((N, F)).astype(np.float32)
    hmap = random_hmap(rng, R, 0.3)
    hbuf = rng.standard_normal((R, F)).astype(np.float32)
    out = orc.fwd_mean_row(ptr, idx, vin, hmap, hbuf)
    np.testing.assert_allclose(out, brute_fwd_mean(ptr, idx, vin, hmap, hbuf), rtol=1e-5, atol=1e-6)
    # closed form D^-1 A X on the non-history rows
    A = sp.csr_matrix((np.ones(len(idx)), idx, ptr), shape=(R, N))
    deg = np.diff(ptr)
    ref = (A @ vin.astype(np.float64)) / np.maximum(deg, 1)[:, None]
    nh = hmap == -1
    np.testing.assert_allclose(out[nh], ref[nh], rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(out[~nh], hbuf[~nh])
    assert (out[nh & (deg == 0)] == 0).all()


def test_fwd_mean_invariants(orc):
    rng = np.random.default_rng(3)
    R, N, F = 30, 20, 16
    ptr, idx = random_csr(rng, R, N, 6)
    vin = rng.standard_normal((N, F)).astype(np.float32)
    hbuf = rng.standard_normal((R, F + 3)).astype(np.float32)  # hsize > F
    none = orc.fwd_mean_row(ptr, idx, vin, None, None)
    all_miss = orc.fwd_mean_row(ptr, idx, vin, np.full(R, -1, np.int64), hbuf)
    np.testing.assert_array_equal(none, all_miss)
    all_hit = orc.fwd_mean_row(ptr, idx, vin, np.zeros(R, np.int64), hbuf)
    np.testing.assert_array_equal(all_hit, hbuf[:, :F])
    # num_node restricts the rows
    part = orc.fwd_mean_row(ptr, idx, vin, None, None, num_node=11)
    np.testing.assert_array_equal(part, none[:11])
    # the independently written PyTorch CPU path agrees
    from oracle import torch_cpu_path as tp
    t = tp.aggr_fwd_row(torch.from_numpy(vin), torch.from_numpy(ptr), torch.from_numpy(idx), None, None, R)
    np.testing.assert_allclose(none, t.numpy(), rtol=1e-5, atol=1e-6)


def test_fwd_src_mode(orc):
    rng = np.random.default_rng(4)
    R, N, F = 25, 40, 12
    ptr, idx = random_csr(rng, R, N, 7)
    feat = rng.standard_normal((N, F)).astype(np.float32)
    hist = rng.standard_normal((17, F)).astype(np.float32)
    hmap = np.full(N, -1, np.int64)
    hit = rng.random(N) < 0.4
    hmap[hit] = rng.integers(0, 17, size=int(hit.sum()))
    out = orc.fwd_mean_src(ptr, idx, feat, hmap, hist)
    # closed form: substitute the table first, then plain mean
    sub = feat.copy()
    sub[hit] = hist[hmap[hit]]
    np.testing.assert_array_equal(out, orc.fwd_mean_row(ptr, idx, sub, None, None))
    np.testing.assert_array_equal(orc.fwd_mean_src(ptr, idx, feat, np.full(N, -1, np.int64), hist),
                                  orc.fwd_mean_row(ptr, idx, feat, None, None))
    from oracle import torch_cpu_path as tp
    t = tp.aggr_fwd_src(torch.from_numpy(feat), torch.from_numpy(hist), torch.from_numpy(hmap),
                        torch.from_numpy(ptr), torch.from_numpy(idx), R)
    np.testing.assert_allclose(out, t.numpy(), rtol=1e-5, atol=1e-6)


def test_bwd_src_mode_routes_gradients_like_autograd(orc):
    """Per-source substitution, backward: pinned by torch autograd of the dense fp64 statement
    out = D^-1 A where(hit, hist[hmap], feat).  A substituted source leaves feat.grad[s] = 0 and sends
    its share to hist.grad[hmap[s]]; table rows shared by several sources add up."""
    rng = np.random.default_rng(41)
    R, N, F, Hn = 30, 40, 8, 9
    ptr, idx = random_csr(rng, R, N, 7)
    hmap = np.full(N, -1, np.int64)
    hit = rng.random(N) < 0.5
    hmap[hit] = rng.integers(0, Hn, size=int(hit.sum()))        # 20 sources onto 9 rows: rows are shared
    g = rng.standard_normal((R, F)).astype(np.float32)
    feat = torch.from_numpy(rng.standard_normal((N, F))).requires_grad_(True)
    hist = torch.from_numpy(rng.standard_normal((Hn, F))).requires_grad_(True)
    hm = torch.from_numpy(hmap)
    rows = torch.where((hm != -1)[:, None], hist[hm.clamp(min=0)], feat)
    deg = np.diff(ptr)
    A = torch.zeros(R, N, dtype=torch.float64)
    for r in range(R):
        for j in range(ptr[r], ptr[r + 1]):
            A[r, idx[j]] += 1.0 / deg[r]
    (A @ rows).backward(torch.from_numpy(g).double())
    gf, gh = orc.bwd_mean_src(ptr, idx, g, N, hmap_src=hmap, hist_shape=(Hn, F))
    np.testing.assert_allclose(gf, feat.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gh, hist.grad.numpy(), rtol=1e-5, atol=1e-6)
    assert (gf[hit] == 0).all() and np.abs(gh).sum() > 0
    # without a map: the gradient of whichever row was read
    np.testing.assert_allclose(orc.bwd_mean_src(ptr, idx, g, N), (A.T @ torch.from_numpy(g).double()).numpy(),
                               rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("seed", [5, 6])
def test_bwd_mean_closed_form_and_adjoint(orc, seed):
    rng = np.random.default_rng(seed)
    R, N, F = 45, 35, 20
    ptr, idx = random_csr(rng, R, N, 8)
    hmap = random_hmap(rng, R, 0.25)
    g = rng.standard_normal((R, F)).astype(np.float32)
    gx, gh = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F))
    deg = np.diff(ptr)
    nh = hmap == -1
    A = sp.csr_matrix((np.ones(len(idx)), idx, ptr), shape=(R, N))
    W = sp.diags(nh / np.maximum(deg, 1)) @ A            # (D^-1 A) with history rows removed
    np.testing.assert_allclose(gx, W.T @ g.astype(np.float64), rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(gh, g * (~nh)[:, None])
    # adjoint identity <fwd(x), g> == <x, bwd_x(g)> + <hbuf, bwd_h(g)>
    x = rng.standard_normal((N, F)).astype(np.float32)
    hbuf = rng.standard_normal((R, F)).astype(np.float32)
    y = orc.fwd_mean_row(ptr, idx, x, hmap, hbuf)
    lhs = (y.astype(np.float64) * g).sum()
    rhs = (x.astype(np.float64) * gx).sum() + (hbuf.astype(np.float64) * gh).sum()
    assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))
    from oracle import torch_cpu_path as tp
    tgx, tgh = tp.aggr_bwd_row(torch.from_numpy(g), torch.from_numpy(ptr), torch.from_numpy(idx),
                               torch.from_numpy(hmap), N, R)
    np.testing.assert_allclose(gx, tgx.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(gh, tgh.numpy())


def test_bwd_matches_autograd_of_dense_formula(orc):
    """d/dx of sum(fwd(x) * g) computed by torch autograd on a dense fp64 statement of the op."""
    rng = np.random.default_rng(7)
    R, N, F = 12, 9, 5
    ptr, idx = random_csr(rng, R, N, 4)
    hmap = random_hmap(rng, R, 0.3)
    x = torch.tensor(rng.standard_normal((N, F)), dtype=torch.float64, requires_grad=True)
    hb = torch.tensor(rng.standard_normal((R, F)), dtype=torch.float64, requires_grad=True)
    g = rng.standard_normal((R, F))
    rows = []
    for r in range(R):
        nb = idx[ptr[r]:ptr[r + 1]]
        if hmap[r] != -1:
            rows.append(hb[r])
        elif len(nb) == 0:
            rows.append(torch.zeros(F, dtype=torch.float64))
        else:
            rows.append(x[torch.from_numpy(nb)].sum(0) / len(nb))
    (torch.stack(rows) * torch.from_numpy(g)).sum().backward()
    gx, gh = orc.bwd_mean_row(ptr, idx, g.astype(np.float32), hmap, N, hbuf_shape=(R, F))
    np.testing.assert_allclose(gx, x.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gh, hb.grad.numpy(), rtol=1e-5, atol=1e-6)


def test_edge_value_closed_forms(orc):
    rng = np.random.default_rng(8)
    R, N, F = 30, 25, 18
    ptr, idx = random_csr(rng, R, N, 6)
    E = len(idx)
    ev = rng.standard_normal(E).astype(np.float32)
    vin = rng.standard_normal((N, F)).astype(np.float32)
    hmap = random_hmap(rng, R, 0.2)
    hbuf = rng.standard_normal((R, F)).astype(np.float32)
    out = orc.fwd_edge_value(ptr, idx, ev, vin, hmap, hbuf)
    A = sp.csr_matrix((ev.astype(np.float64), idx, ptr), shape=(R, N))
    nh = hmap == -1
    np.testing.assert_allclose(out[nh], (A @ vin.astype(np.float64))[nh], rtol=1e-4, atol=1e-5)
    np.testing.assert_array_equal(out[~nh], hbuf[~nh])
    # ev == 1/deg reproduces the mean on non-empty rows
    deg = np.diff(ptr)
    inv = np.repeat(1.0 / np.maximum(deg, 1), deg).astype(np.float32)
    m = orc.fwd_mean_row(ptr, idx, vin, None, None)
    w = orc.fwd_edge_value(ptr, idx, inv, vin, None, None)
    np.testing.assert_allclose(w, m, rtol=1e-5, atol=1e-6)
    # backward: weighted transpose product, SDDMM for edge_grad
    g = rng.standard_normal((R, F)).astype(np.float32)
    gx, gh, eg = orc.bwd_edge_value(ptr, idx, ev, g, hmap, vin, N, hsize=F, want_edge_grad=True)
    Anh = sp.diags(nh.astype(np.float64)) @ A
    np.testing.assert_allclose(gx, Anh.T @ g.astype(np.float64), rtol=1e-4, atol=1e-5)
    np.testing.assert_array_equal(gh, g * (~nh)[:, None])
    dst = np.repeat(np.arange(R), deg)
    sddmm = (g[dst].astype(np.float64) * vin[idx].astype(np.float64)).sum(1) * nh[dst]
    np.testing.assert_allclose(eg, sddmm, rtol=1e-5, atol=1e-6)


def test_multi_head_reductions(orc):
    rng = np.random.default_rng(9)
    R, N, F, H = 20, 15, 6, 3
    ptr, idx = random_csr(rng, R, N, 5)
    E = len(idx)
    vin = rng.standard_normal((N, H, F)).astype(np.float32)
    ev = rng.standard_normal((E, H)).astype(np.float32)
    hmap = random_hmap(rng, R, 0.3)
    hb_shared = rng.standard_normal((R, F)).astype(np.float32)
    hb_cat = rng.standard_normal((R, F * H)).astype(np.float32)
    out_s = orc.fwd_edge_value(ptr, idx, ev, vin, hmap, hb_shared)
    out_c = orc.fwd_edge_value(ptr, idx, ev, vin, hmap, hb_cat)
    for h in range(H):
        single = orc.fwd_edge_value(ptr, idx, np.ascontiguousarray(ev[:, h]),
                                    np.ascontiguousarray(vin[:, h]), hmap, hb_shared)
        np.testing.assert_array_equal(out_s[:, h], single)
        nh = hmap == -1
        np.testing.assert_array_equal(out_c[nh, h], single[nh])
        np.testing.assert_array_equal(out_c[~nh, h], hb_cat[~nh, h * F:(h + 1) * F])
    g = rng.standard_normal((R, H, F)).astype(np.float32)
    gx, gh, eg = orc.bwd_edge_value(ptr, idx, ev, g, hmap, vin, N, hsize=F, want_edge_grad=True)
    gx2, gh2, _ = orc.bwd_edge_value(ptr, idx, ev, g, hmap, vin, N, hsize=F * H)
    for h in range(H):
        sx, sh, se = orc.bwd_edge_value(ptr, idx, np.ascontiguousarray(ev[:, h]),
                                        np.ascontiguousarray(g[:, h]), hmap,
                                        np.ascontiguousarray(vin[:, h]), N, hsize=F, want_edge_grad=True)
        np.testing.assert_array_equal(gx[:, h], sx)
        np.testing.assert_array_equal(eg[:, h], se)
        np.testing.assert_array_equal(gh2[:, h * F:(h + 1) * F], sh)
    np.testing.assert_allclose(gh, g.sum(1) * (hmap != -1)[:, None], rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        orc.fwd_edge_value(ptr, idx, ev, vin, hmap, rng.standard_normal((R, F + 1)).astype(np.float32))


def test_build_transpose_is_stable_sort(orc):
    rng = np.random.default_rng(10)
    R, N = 60, 20
    ptr, idx = random_csr(rng, R, N, 9)
    hmap = random_hmap(rng, R, 0.3)
    ptrT, rowT, edgeT = orc.build_transpose(ptr, idx, hmap, N)
    deg = np.diff(ptr)
    dst = np.repeat(np.arange(R), deg)
    keep = np.flatnonzero(hmap[dst] == -1)
    order = keep[np.argsort(idx[keep], kind="stable")]
    np.testing.assert_array_equal(edgeT, order)
    np.testing.assert_array_equal(rowT, dst[order])
    np.testing.assert_array_equal(ptrT, np.concatenate([[0], np.cumsum(np.bincount(idx[keep], minlength=N))]))


def test_quarter_split_order(orc):
    """split_above restates the device library's long-row order: four contiguous quarters summed
    separately, combined left to right.  Written out independently with NumPy float32."""
    rng = np.random.default_rng(11)
    N, F = 50, 9
    deg = np.array([3, 0, 23, 8, 41])
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    idx = rng.integers(0, N, size=int(ptr[-1]), dtype=np.int64)
    vin = rng.standard_normal((N, F)).astype(np.float32)
    got = orc.fwd_mean_row(ptr, idx, vin, None, None, split_above=8)
    seq = orc.fwd_mean_row(ptr, idx, vin, None, None)
    for r, d in enumerate(deg):
        nb = idx[ptr[r]:ptr[r + 1]]
        if d <= 8:
            np.testing.assert_array_equal(got[r], seq[r])
            continue
        q = -(-d // 4)
        parts = []
        for w in range(4):
            acc = np.zeros(F, np.float32)
            for j in nb[w * q:(w + 1) * q]:
                acc = acc + vin[j]
            parts.append(acc)
        tot = ((parts[0] + parts[1]) + parts[2]) + parts[3]
        np.testing.assert_array_equal(got[r], tot / np.float32(d))
    np.testing.assert_allclose(got, seq, rtol=1e-5, atol=1e-6)
    hist = rng.standard_normal((7, F)).astype(np.float32)
    hm = np.where(rng.random(N) < 0.5, rng.integers(0, 7, size=N), -1).astype(np.int64)
    sub = vin.copy()
    sub[hm != -1] = hist[hm[hm != -1]]
    np.testing.assert_array_equal(orc.fwd_mean_src(ptr, idx, vin, hm, hist, split_above=8),
                                  orc.fwd_mean_row(ptr, idx, sub, None, None, split_above=8))


def test_chunked_backward_order(orc):
    """chunk > 0 restates the device order for hub sources: chunks of `chunk` incoming edges summed
    from zero, chunk sums combined left to right.  Written out independently with NumPy float32."""
    rng = np.random.default_rng(12)
    R, N, F, C = 60, 6, 5, 8
    deg = rng.integers(1, 5, size=R)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    idx = rng.integers(0, N, size=int(ptr[-1]), dtype=np.int64)
    idx[idx == 4] = 5                                   # source 4 has no edges
    g = rng.standard_normal((R, F)).astype(np.float32)
    hmap = np.where(rng.random(R) < 0.2, 3, -1).astype(np.int64)
    got, _ = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F), chunk=C)
    seq, _ = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, F))
    dst = np.repeat(np.arange(R), deg)
    for s in range(N):
        es = [e for e in range(len(idx)) if idx[e] == s and hmap[dst[e]] == -1]
        terms = [g[dst[e]] / np.float32(deg[dst[e]]) for e in es]
        if len(es) <= C:
            np.testing.assert_array_equal(got[s], seq[s])
            continue
        tot = None
        for c0 in range(0, len(terms), C):
            acc = np.zeros(F, np.float32)
            for t in terms[c0:c0 + C]:
                acc = acc + t
            tot = acc if tot is None else tot + acc
        np.testing.assert_array_equal(got[s], tot)
    np.testing.assert_allclose(got, seq, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("seed,R_layer", [(21, 25), (22, 60), (23, 1), (24, 0)])
def test_batch_view_backward_order(orc, seed, R_layer):
    """The summation order over ONE view of the whole mini-batch CSR (hc_aggr_bwd_batch_view): positions
    count every edge of the batch's rows, a hub is a source with more than `chunk` of them, a chunk is a
    run of `chunk` positions of which only the live edges (rows of the layer that did not take their
    history row) are added.  Written out independently with NumPy float32; equal, as a value, to the
    dense product in fp64; the same bits as the per-layer statement wherever no hub is involved."""
    rng = np.random.default_rng(seed)
    R_all, N, F, C = 60, 9, 5, 8
    deg = rng.integers(0, 5, size=R_all)
    ptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    idx = rng.integers(0, N, size=int(ptr[-1]), dtype=np.int64)
    idx[idx == 4] = 5                                   # source 4 has no edges
    n_src = 7                                           # the layer's sources; rows of the layer stay below
    dst = np.repeat(np.arange(R_all), deg)
    idx[(dst < R_layer) & (idx >= n_src)] = 1
    g = rng.standard_normal((R_layer, F)).astype(np.float32)
    hmap = np.where(rng.random(R_layer) < 0.3, 3, -1).astype(np.int64)
    got, gh = orc.bwd_mean_row_batch_view(ptr, idx, g, hmap, n_src, R_all, hbuf_shape=(R_layer, F), chunk=C)
    seq, gh_seq = orc.bwd_mean_row(ptr[:R_layer + 1], idx, g, hmap, n_src, hbuf_shape=(R_layer, F))
    np.testing.assert_array_equal(gh, gh_seq)
    unchunked, _ = orc.bwd_mean_row_batch_view(ptr, idx, g, hmap, n_src, R_all, hbuf_shape=(R_layer, F))
    np.testing.assert_array_equal(unchunked, seq)       # without a chunk rule the view's extent is irrelevant
    live = lambda e: dst[e] < R_layer and hmap[dst[e]] == -1
    any_hub = False
    for s in range(n_src):
        es = [e for e in range(len(idx)) if idx[e] == s]            # view positions: (row, slot) ascending
        if len(es) <= C:
            np.testing.assert_array_equal(got[s], seq[s])
            continue
        any_hub = True
        tot = None
        for c0 in range(0, len(es), C):
            acc = np.zeros(F, np.float32)
            for e in es[c0:c0 + C]:
                if live(e):
                    acc = acc + g[dst[e]] / np.float32(deg[dst[e]])
            tot = acc if tot is None else tot + acc
        np.testing.assert_array_equal(got[s], tot)
    assert any_hub
    # value: (D^-1 A restricted to live rows)^T g in fp64
    A = sp.csr_matrix((np.ones(int(ptr[R_layer])), idx[:ptr[R_layer]], ptr[:R_layer + 1]), shape=(R_layer, N))
    scale = (hmap == -1) / np.maximum(deg[:R_layer], 1)
    ref = (A.T @ (g.astype(np.float64) * scale[:, None]))[:n_src]
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_multithreaded_cpu_statement_equals_the_sequential_one(orc):
    """The OpenMP statement that the benchmark times as its CPU baseline gives the sequential statement's
    bits: forward with per-source substitution (long rows as quarters), transposed view, backward gather
    (hub sources in chunks)."""
    from oracle import hc_cpu_mt as mt
    assert mt.num_threads() >= 1
    rng = np.random.default_rng(77)
    for R, N, F, hub in [(3000, 2000, 64, 1500), (500, 40, 17, None), (1, 1, 8, None), (257, 5000, 256, 300)]:
        ptr, idx = random_csr(rng, R, N, 12, hub=hub)
        idx[rng.random(len(idx)) < 0.2] = N // 3                    # one very popular source
        feat = rng.standard_normal((N, F)).astype(np.float32)
        hist = rng.standard_normal((50, F)).astype(np.float32)
        smap = np.where(rng.random(N) < 0.4, rng.integers(0, 50, size=N), -1).astype(np.int64)
        for m, h in ((smap, hist), (None, None)):
            np.testing.assert_array_equal(mt.fwd_mean_src(ptr, idx, feat, m, h, split_above=256),
                                          orc.fwd_mean_src(ptr, idx, feat, m, h, split_above=256))
        ptrT, rowT = mt.build_transpose(ptr, idx, N)
        wp, wr, _ = orc.build_transpose(ptr, idx, None, N)
        np.testing.assert_array_equal(ptrT, wp)
        np.testing.assert_array_equal(rowT[: len(wr)], wr)
        g = rng.standard_normal((R, F)).astype(np.float32)
        for chunk in (0, 512):
            np.testing.assert_array_equal(mt.bwd_mean(ptr, ptrT, rowT, g, N, chunk=chunk),
                                          orc.bwd_mean_src(ptr, idx, g, N, chunk=chunk))
        # the view without the substituted sources: their gradient rows are zero, the others keep their bits
        ptrS, rowS = mt.build_transpose(ptr, idx, N, hmap_src=smap)
        np.testing.assert_array_equal(np.diff(ptrS), np.where(smap == -1, np.diff(ptrT), 0))
        np.testing.assert_array_equal(mt.bwd_mean(ptr, ptrS, rowS, g, N, chunk=512),
                                      orc.bwd_mean_src(ptr, idx, g, N, chunk=512, hmap_src=smap)[0])
    with pytest.raises(ValueError):
        mt.build_transpose(np.array([0, 1]), np.array([5]), 3)
