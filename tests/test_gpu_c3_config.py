"""The papers100M-shaped configuration at its stated batch shape: 3-layer GraphSAGE, hidden 256,
128-dim fp32 features read zero-copy from pinned host memory, 172 classes, fanout [15, 10, 5],
1000 seeds, fp16 ring history table with about 35% of the nodes cached.  The graph (power-law
out-degrees, popular targets) is cut to 600 000 nodes so that the CPU side can hold it, and the
table to one row per node of that graph; everything a batch touches has the configuration's shape.
One iteration of sampling -> lookup_and_load -> forward/backward -> admission on the GPU against
the CPU statements: indices, masks, maps and stored rows exactly, logits and gradients within the
fp32 tolerances of the plumbing configuration's test."""
import numpy as np
import pytest
import torch

from helpers import power_law_graph
from test_gpu_cache import CpuSage

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("emit_view", [False, True])
def test_c3_iteration_matches_cpu(orc, emit_view, monkeypatch):
    """``emit_view``: the sampler hands the batch over together with the transposed view of its CSR and
    the layers' backward builds none (the call is made to fail inside backward)."""
    from hiscache import HistorySAGE, NeighborSampler, PinnedFeatureStore, RingHistoryCache, make_config
    from hiscache.synthetic import make_batch
    from oracle import host_model
    N, F, H, C, L, n_seed, fanout = 600_000, 128, 256, 172, 3, 1000, [15, 10, 5]
    rng = np.random.default_rng(3)
    torch.manual_seed(3)
    indptr, indices = power_law_graph(rng, N, 2.6, alpha=2.0)
    feats = rng.standard_normal((N, F), dtype=np.float32)
    labels = rng.integers(0, C, size=N)
    cached = rng.permutation(N)[: int(0.35 * N)]
    rows16 = (0.5 * rng.standard_normal((len(cached), H), dtype=np.float32)).astype(np.float16)

    cache = RingHistoryCache(PinnedFeatureStore(torch.from_numpy(feats), device=DEV), N, F, H, capacity=N,
                             num_layers=L, table_dtype=torch.float16, rate=0.5, age_limit=200, device=DEV)
    cache.preload(torch.from_numpy(cached).to(DEV), torch.from_numpy(rows16).to(DEV))
    ref = dict(table=np.zeros((N, H), np.uint16), f2s=np.full(N, -1, np.int64), s2f=np.full(N, -1, np.int64),
               checkin=np.full(N, -1, np.int64), header=np.array([len(cached)], np.int64))
    ref["table"][: len(cached)] = rows16.view(np.uint16)
    ref["f2s"][cached] = np.arange(len(cached))
    ref["s2f"][: len(cached)] = cached
    ref["checkin"][: len(cached)] = 0

    # --- sampling: device sampler against the sequential statement
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=3, device=DEV, emit_view=emit_view)
    seeds = rng.choice(N, size=n_seed, replace=False).astype(np.int64)
    batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
    b = orc.sample_layers(indptr, indices, seeds, fanout, sampler.batch_seed(0))
    for k, got in (("ptr", batch.ptr), ("idx", batch.idx), ("sub_to_full", batch.sub_to_full)):
        np.testing.assert_array_equal(got.cpu().numpy(), b[k])
    nnl = b["num_node_in_layer"]
    n1, n2, n_all = int(nnl[1]), int(nnl[2]), int(nnl[3])
    assert nnl[0] == 1000 and 3000 < n1 <= 16_000 and n2 <= 176_000 and n_all <= 1_060_000
    assert list(batch.num_edge_in_layer) == [int(b["ptr"][int(nnl[k])]) for k in range(L)]

    # --- lookup_and_load: slots, used masks, loaded rows, cached rows
    cache.lookup_and_load(batch, L)
    tab32 = ref["table"].view(np.float16).astype(np.float32)
    slot, hbuf = host_model.ring_lookup(ref["f2s"], ref["checkin"], b["sub_to_full"][:n1], 1, 200, tab32)
    np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), slot)
    np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), hbuf)
    used = orc.count_history_reconstruct(b["ptr"], b["idx"], slot, n_all, n_seed, L)
    assert len(cache.used_masks) == L + 1
    for got, want in zip(cache.used_masks, used):
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    x_ref = feats[b["sub_to_full"]] * used[0][:, None]
    np.testing.assert_array_equal(batch.x.cpu().numpy(), x_ref)
    hit = slot != -1
    assert 0.25 < hit.mean() < 0.45
    assert used[0].sum() < n_all               # the cached 1-hop nodes prune part of the sub-tree

    # --- model forward / backward
    cfg = make_config(F, C, H, L, device=DEV)
    model = HistorySAGE(F, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
    model.train()
    cpu_model = CpuSage(model)
    cpu_model.m.train()
    seen = {}
    hook = model.convs[L - 2].register_forward_pre_hook(lambda mod, args: seen.__setitem__("x", args[0].detach()))
    out = model(batch)
    hook.remove()
    loss = torch.nn.functional.nll_loss(out, batch.y)
    assert (batch.view is not None) == emit_view
    if emit_view:
        import hiscache_backend

        def no_view_in_backward(*a, **k):
            raise AssertionError("a transposed view was built inside backward")
        monkeypatch.setattr(hiscache_backend, "build_transpose", no_view_in_backward)
    loss.backward()
    monkeypatch.undo()
    pe = cache.produced_embedding
    assert tuple(pe.shape) == (n1, H)
    # the history layer's output from the GPU's own layer-1 activations, bit for bit
    want_pe = orc.fwd_mean_row(b["ptr"], b["idx"], seen["x"].cpu().numpy(), slot, hbuf, n1)
    np.testing.assert_array_equal(pe.detach().cpu().numpy(), want_pe)
    cpu_batch = make_batch(b, labels, "cpu")
    out_c, his_c = cpu_model(cpu_batch, torch.from_numpy(x_ref), torch.from_numpy(slot), torch.from_numpy(hbuf))
    loss_c = torch.nn.functional.nll_loss(out_c, cpu_batch.y)
    loss_c.backward()
    np.testing.assert_allclose(out.detach().cpu().numpy(), out_c.detach().numpy(), rtol=1e-4, atol=2e-5)
    gs = float(his_c.grad.abs().max())
    np.testing.assert_allclose(pe.grad.cpu().numpy(), his_c.grad.numpy(), rtol=1e-3, atol=1e-5 * gs)
    gscale = max(float(q.grad.abs().max()) for q in cpu_model.m.parameters() if q.grad is not None)
    for (name, p), (_, q) in zip(model.named_parameters(), cpu_model.m.named_parameters()):
        if p.grad is not None:
            # weight gradients are fp32 sums over up to 60 000 rows, in another order on the CPU: 1e-3 relative,
            # with an absolute floor of 2e-4 of the largest gradient for the near-zero entries
            np.testing.assert_allclose(p.grad.cpu().numpy(), q.grad.numpy(), rtol=1e-3, atol=2e-4 * gscale,
                                       err_msg=name)

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
