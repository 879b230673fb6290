"""The CPU-runnable plumbing configuration at its stated shape: uniform graph of 100k nodes (mean
out-degree 15), 128-dim fp32 features, 10 classes, 2-layer SAGE hidden 128, 1000 seeds, fanout
[10, 5], history table 100k x 128 fp32 with a random 30% of the nodes cached.  One iteration of
sampling -> lookup_and_load -> history aggregation forward/backward -> admission on the GPU against
the CPU statements."""
import numpy as np
import pytest
import torch

from test_gpu_cache import CpuSage

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_c1_iteration_matches_cpu(orc):
    from hiscache import HistorySAGE, NeighborSampler, PinnedFeatureStore, RingHistoryCache, make_config
    from hiscache.synthetic import make_batch, uniform_graph
    from oracle import host_model
    N, F, H, C, L, n_seed, fanout = 100_000, 128, 128, 10, 2, 1000, [10, 5]
    rng = np.random.default_rng(1)
    torch.manual_seed(1)
    indptr, indices = uniform_graph(N, 15, 1)
    feats = rng.standard_normal((N, F)).astype(np.float32)
    labels = rng.integers(0, C, size=N)
    cached = rng.permutation(N)[: int(0.3 * N)]
    rows = rng.standard_normal((len(cached), H)).astype(np.float32)

    cache = RingHistoryCache(PinnedFeatureStore(torch.from_numpy(feats), device=DEV), N, F, H, capacity=N,
                             num_layers=L, table_dtype=torch.float32, rate=0.5, age_limit=1 << 30, device=DEV)
    cache.preload(torch.from_numpy(cached).to(DEV), torch.from_numpy(rows).to(DEV))
    ref = dict(table=np.zeros((N, H), np.float32), f2s=np.full(N, -1, np.int64), s2f=np.full(N, -1, np.int64),
               checkin=np.full(N, -1, np.int64), header=np.array([len(cached)], np.int64))
    ref["table"][: len(cached)] = rows
    ref["f2s"][cached] = np.arange(len(cached))
    ref["s2f"][: len(cached)] = cached
    ref["checkin"][: len(cached)] = 0

    # --- sampling: device sampler against the sequential statement
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=1, device=DEV)
    seeds = rng.choice(N, size=n_seed, replace=False).astype(np.int64)
    batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
    b = orc.sample_layers(indptr, indices, seeds, fanout, sampler.batch_seed(0))
    for k, got in (("ptr", batch.ptr), ("idx", batch.idx), ("sub_to_full", batch.sub_to_full)):
        np.testing.assert_array_equal(got.cpu().numpy(), b[k])
    nnl = b["num_node_in_layer"]
    n1 = int(nnl[1])
    assert nnl[0] == 1000 and 5000 < n1 <= 11_000 and nnl[2] <= 66_000

    # --- lookup_and_load
    cache.lookup_and_load(batch, L)
    slot = ref["f2s"][b["sub_to_full"][:n1]]
    np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), slot)
    used = orc.count_history_reconstruct(b["ptr"], b["idx"], slot, int(nnl[2]), n_seed, L)
    for got, want in zip(cache.used_masks, used):
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    x_ref = feats[b["sub_to_full"]] * used[0][:, None]
    np.testing.assert_array_equal(batch.x.cpu().numpy(), x_ref)
    hit = slot != -1
    assert 0.2 < hit.mean() < 0.4
    np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy()[hit], ref["table"][slot[hit]])

    # --- model forward / backward
    cfg = make_config(F, C, H, L, device=DEV)
    model = HistorySAGE(F, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
    model.train()
    cpu_model = CpuSage(model)
    cpu_model.m.train()
    out = model(batch)
    loss = torch.nn.functional.nll_loss(out, batch.y)
    loss.backward()
    pe = cache.produced_embedding
    # the history layer's output, bit for bit
    hbuf = cache.cached_embedding.cpu().numpy()
    want_pe = orc.fwd_mean_row(b["ptr"], b["idx"], x_ref, slot, hbuf, n1)
    np.testing.assert_array_equal(pe.detach().cpu().numpy(), want_pe)
    cpu_batch = make_batch(b, labels, "cpu")
    out_c, his_c = cpu_model(cpu_batch, torch.from_numpy(x_ref), torch.from_numpy(slot), torch.from_numpy(hbuf))
    loss_c = torch.nn.functional.nll_loss(out_c, cpu_batch.y)
    loss_c.backward()
    np.testing.assert_allclose(out.detach().cpu().numpy(), out_c.detach().numpy(), rtol=1e-4, atol=1e-5)
    gs = float(his_c.grad.abs().max())
    np.testing.assert_allclose(pe.grad.cpu().numpy(), his_c.grad.numpy(), rtol=1e-3, atol=1e-5 * gs)
    gscale = max(float(q.grad.abs().max()) for q in cpu_model.m.parameters() if q.grad is not None)
    for (name, p), (_, q) in zip(model.named_parameters(), cpu_model.m.named_parameters()):
        if p.grad is not None:
            np.testing.assert_allclose(p.grad.cpu().numpy(), q.grad.numpy(), rtol=1e-3, atol=2e-5 * gscale,
                                       err_msg=name)

    # --- admission on the GPU's own gradient: mask, maps, header and table rows exact
    grad = pe.grad.cpu().numpy()
    emb = pe.detach().cpu().numpy()
    cache.update_history(batch, 1)
    score = orc.row_scores(grad)
    thres = float(host_model.quantile_threshold(score, 0.5))
    age = (1 - ref["checkin"][np.maximum(slot, 0)]).astype(np.int32)
    rmask, _, _ = orc.grad_check(grad, emb, slot, age, None, b["sub_to_full"][:n1], thres, 1 << 30, orc.NORM_L2,
                                 orc.CMP_LT, ref["table"], orc.DT_F32, ref["f2s"], ref["s2f"], ref["checkin"],
                                 ref["header"], 1)
    assert 0 < rmask.sum() < n1
    np.testing.assert_array_equal(cache.last_record_mask.cpu().numpy(), rmask)
    np.testing.assert_array_equal(cache.full2slot.cpu().numpy(), ref["f2s"])
    np.testing.assert_array_equal(cache.slot2full.cpu().numpy(), ref["s2f"])
    np.testing.assert_array_equal(cache.checkin.cpu().numpy(), ref["checkin"])
    assert cache.header == int(ref["header"][0])
    np.testing.assert_array_equal(cache.table.cpu().numpy(), ref["table"])
