"""The mag240M-shaped configuration at its stated batch shape: 2-layer relational GCN, hidden 256, 5
relations derived from the node types of an edge's ends (papers, authors, institutions stored as
consecutive id ranges), 768-dim fp16 paper-style features read zero-copy from pinned host memory,
153 classes, fanout [25, 15], 1000 seeds, fp16 ring history table with about 35% of the nodes
cached.  The graph is cut to 300 000 nodes (power-law out-degrees, popular targets) so that the CPU
side can hold it.  One iteration of sampling -> lookup_and_load -> forward/backward -> admission on
the GPU: indices, relations, (row, relation) groups, masks, maps and stored rows exactly; the
relational convolution against a dense fp64 statement sum_j x[src_j] W[rel_j] / deg."""
import numpy as np
import pytest
import torch

from helpers import power_law_graph

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rgcn_layer_fp64(x, W, ptr, idx, rel, used, n, hit=None, hbuf=None):
    """sum_j x[src_j] @ W[rel_j] / deg over the first n rows in fp64, one relation at a time; sources
    outside ``used`` are dropped, rows flagged by ``hit`` take their cached row."""
    deg = ptr[1:n + 1] - ptr[:n]
    E = int(ptr[n])
    dst = torch.repeat_interleave(torch.arange(n), deg)
    src = idx[:E]
    keep = used[src] if used is not None else torch.ones(E, dtype=torch.bool)
    out = torch.zeros(n, W.shape[2], dtype=torch.float64)
    for k in range(W.shape[0]):
        m = keep & (rel[:E] == k)
        agg = torch.zeros(n, x.shape[1], dtype=torch.float64).index_add(0, dst[m], x[src[m]].double())
        out = out + agg @ W[k].double()
    out = out / deg.clamp(min=1).double()[:, None]
    if hit is not None:
        out = torch.where(hit[:, None], hbuf.double(), out)
    return out


@pytest.mark.parametrize("emit_view", [False, True])
def test_c5_iteration_matches_cpu(orc, emit_view, monkeypatch):
    """``emit_view``: the sampler hands the batch over together with the transposed view of its CSR (with
    edge slots) and the relational layer's backward builds none (the call is made to fail inside backward)."""
    from hiscache import HistoryRGCN, NeighborSampler, PinnedFeatureStore, RingHistoryCache, make_config
    from oracle import host_model
    n_paper, n_author, n_inst = 150_000, 147_000, 3_000
    N = n_paper + n_author + n_inst
    F, H, C, K, L, n_seed, fanout = 768, 256, 153, 5, 2, 1000, [25, 15]
    rng = np.random.default_rng(5)
    torch.manual_seed(5)
    indptr, indices = power_law_graph(rng, N, 1.25, alpha=2.0)
    feats16 = rng.standard_normal((N, F), dtype=np.float32).astype(np.float16)
    labels = rng.integers(0, C, size=N)
    cached = rng.permutation(N)[: int(0.35 * N)]
    rows16 = (0.5 * rng.standard_normal((len(cached), H), dtype=np.float32)).astype(np.float16)

    store = PinnedFeatureStore(torch.from_numpy(feats16), device=DEV, out_dtype=torch.float16)
    cache = RingHistoryCache(store, N, F, H, capacity=N, num_layers=L, table_dtype=torch.float16, rate=0.5,
                             age_limit=200, device=DEV)
    cache.preload(torch.from_numpy(cached).to(DEV), torch.from_numpy(rows16).to(DEV))
    ref = dict(table=np.zeros((N, H), np.uint16), f2s=np.full(N, -1, np.int64), s2f=np.full(N, -1, np.int64),
               checkin=np.full(N, -1, np.int64), header=np.array([len(cached)], np.int64))
    ref["table"][: len(cached)] = rows16.view(np.uint16)
    ref["f2s"][cached] = np.arange(len(cached))
    ref["s2f"][: len(cached)] = cached
    ref["checkin"][: len(cached)] = 0

    # --- sampling
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=5, device=DEV, emit_view=emit_view,
                              view_edges=True)
    seeds = rng.choice(n_paper, size=n_seed, replace=False).astype(np.int64)        # seeds are papers
    batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
    b = orc.sample_layers(indptr, indices, seeds, fanout, sampler.batch_seed(0))
    for k, got in (("ptr", batch.ptr), ("idx", batch.idx), ("sub_to_full", batch.sub_to_full)):
        np.testing.assert_array_equal(got.cpu().numpy(), b[k])
    nnl = b["num_node_in_layer"]
    n1, n_all = int(nnl[1]), int(nnl[2])
    assert nnl[0] == 1000 and 2000 < n1 <= 26_000 and n_all <= 416_000

    # --- lookup_and_load
    cache.lookup_and_load(batch, L)
    tab32 = ref["table"].view(np.float16).astype(np.float32)
    slot, hbuf = host_model.ring_lookup(ref["f2s"], ref["checkin"], b["sub_to_full"][:n1], 1, 200, tab32)
    np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), slot)
    np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), hbuf)
    used = orc.count_history_reconstruct(b["ptr"], b["idx"], slot, n_all, n_seed, L)
    for got, want in zip(cache.used_masks, used):
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    assert batch.x.dtype == torch.float16
    x_ref16 = np.where(used[0][:, None], feats16[b["sub_to_full"]], np.float16(0))
    np.testing.assert_array_equal(batch.x.cpu().numpy().view(np.uint16), x_ref16.view(np.uint16))
    hit = slot != -1
    assert 0.25 < hit.mean() < 0.45 and used[0].sum() < n_all

    # --- relations and (row, relation) groups of the first layer, exact
    cfg = make_config(F, C, H, L, device=DEV, model_type="rgcn", num_rel=K, name="rmag240m")
    pair_to_rel = [[0, 1, 0], [2, 0, 3], [0, 4, 0]]
    bounds = [n_paper, n_paper + n_author]
    model = HistoryRGCN(F, H, C, L, 0.0, "CSR_Layer", cfg, cache, num_rel=K, dataset_name="rmag240m",
                        type_bounds=bounds, pair_to_rel=pair_to_rel).to(DEV)
    model.train()
    et = model.edge_types(batch)
    want_et = orc.edge_types_by_ranges(b["ptr"], b["idx"], b["sub_to_full"], n1, np.array(bounds),
                                       np.array(pair_to_rel))
    np.testing.assert_array_equal(et.cpu().numpy(), want_et)
    assert set(np.unique(want_et[: int(b["ptr"][n1])])) == {0, 1, 2, 3, 4}
    import hiscache_backend as be
    e1 = int(b["ptr"][n1])
    got_t = be.typed_csr(batch.ptr, batch.idx, et[:e1].contiguous(), K, n1, n_all, cache.used_masks[0])
    want_t = orc.typed_csr(b["ptr"], b["idx"], want_et[:e1], K, n1, n_all, used[0])
    np.testing.assert_array_equal(got_t[0].cpu().numpy(), want_t[0])
    np.testing.assert_array_equal(got_t[1].cpu().numpy()[: want_t[0][-1]], want_t[1])
    np.testing.assert_array_equal(got_t[2].cpu().numpy(), want_t[2])
    np.testing.assert_array_equal(got_t[3].cpu().numpy(), want_t[3])

    # --- model forward / backward against the dense fp64 statement
    out = model(batch)
    loss = torch.nn.functional.nll_loss(out, batch.y)
    assert (batch.view is not None) == emit_view
    if emit_view:
        def no_view_in_backward(*a, **k):
            raise AssertionError("a transposed view was built inside backward")
        monkeypatch.setattr(be, "build_transpose", no_view_in_backward)
    loss.backward()
    monkeypatch.undo()
    np.testing.assert_array_equal(model.convs[0].last_count.cpu().numpy(), orc.count_num(want_et[:e1], K))
    ptr, idx = torch.from_numpy(b["ptr"]), torch.from_numpy(b["idx"])
    rel = torch.from_numpy(want_et)
    W0 = model.convs[0].linear.detach().cpu().double().requires_grad_(True)
    W1 = model.convs[1].linear.detach().cpu().double().requires_grad_(True)
    x0 = torch.from_numpy(x_ref16.astype(np.float32))
    um = [torch.from_numpy(u) for u in used]
    h1 = rgcn_layer_fp64(x0, W0, ptr, idx, rel, um[0], n1, torch.from_numpy(hit), torch.from_numpy(hbuf))
    h1.retain_grad()
    bn = model.bns[0]
    mu, var = h1.mean(0), h1.var(0, unbiased=False)
    z = (h1 - mu) / torch.sqrt(var + bn.eps) * bn.weight.detach().cpu().double() + bn.bias.detach().cpu().double()
    z = torch.relu(z)
    o = rgcn_layer_fp64(z, W1, ptr, idx, rel, um[-2], n_seed).log_softmax(dim=-1)
    loss_c = torch.nn.functional.nll_loss(o, batch.y.cpu())
    loss_c.backward()
    pe = cache.produced_embedding
    assert tuple(pe.shape) == (n1, H)
    # rows with a cached embedding carry it exactly; the computed rows match the fp64 statement
    np.testing.assert_array_equal(pe.detach().cpu().numpy()[hit], hbuf[hit])
    np.testing.assert_allclose(pe.detach().cpu().numpy(), h1.detach().numpy(), rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(out.detach().cpu().numpy(), o.detach().numpy(), rtol=2e-3, atol=2e-3)
    gs = float(h1.grad.abs().max())
    np.testing.assert_allclose(pe.grad.cpu().numpy(), h1.grad.numpy(), rtol=1e-2, atol=2e-3 * gs)
    for got, want in ((model.convs[0].linear.grad, W0.grad), (model.convs[1].linear.grad, W1.grad)):
        s = float(want.abs().max())
        np.testing.assert_allclose(got.cpu().numpy(), want.numpy(), rtol=1e-2, atol=2e-3 * s)

    # --- admission on the GPU's own gradient: mask, maps, header and table rows exact
    grad = pe.grad.cpu().numpy()
    emb = pe.detach().cpu().numpy()
    cache.update_history(batch, 1)
    score = orc.row_scores(grad)
    thres = float(host_model.quantile_threshold(score, 0.5))
    rmask, _, _ = orc.grad_check(grad, emb, slot, None, None, b["sub_to_full"][:n1], thres, 0, orc.NORM_L2,
                                 orc.CMP_LT, ref["table"], orc.DT_F16, ref["f2s"], ref["s2f"], ref["checkin"],
                                 ref["header"], 1)
    assert 0 < rmask.sum() < n1 and not (rmask & hit).any()
    np.testing.assert_array_equal(cache.last_record_mask.cpu().numpy(), rmask)
    np.testing.assert_array_equal(cache.full2slot.cpu().numpy(), ref["f2s"])
    np.testing.assert_array_equal(cache.slot2full.cpu().numpy(), ref["s2f"])
    np.testing.assert_array_equal(cache.checkin.cpu().numpy(), ref["checkin"])
    assert cache.header == int(ref["header"][0])
    np.testing.assert_array_equal(cache.table.view(torch.int16).cpu().numpy().view(np.uint16), ref["table"])
