"""End to end: a few dozen iterations of the training loop (device sampler -> lookup_and_load -> model ->
optimizer -> admission) on a task whose labels follow from the features.  Parity is covered elsewhere;
this checks that the fused layers, the cache and the optimizer work together: the loss falls, the cache
fills and serves hits, and the state stays finite."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("kind", ["sage", "rgcn"])
def test_training_reduces_the_loss(kind):
    losses, hits, model, cache = _train(kind, 90, lambda loss: loss.backward())
    assert all(np.isfinite(losses))
    first, last = float(np.mean(losses[:10])), float(np.mean(losses[-10:]))
    assert last < 0.7 * first, (first, last)
    assert max(hits[30:]) > 0.02                      # admitted rows come back as hits
    assert cache.header > 0
    for p in model.parameters():
        assert bool(torch.isfinite(p).all())
    for name, buf in model.named_buffers():
        if "running" in name:
            assert bool(torch.isfinite(buf).all())
        if "num_batches_tracked" in name:
            assert int(buf) == 90


@pytest.mark.parametrize("kind", ["sage", "rgcn"])
def test_backward_on_the_calling_thread_changes_nothing(kind):
    """hiscache.backward_on_this_thread(loss) (no hand-over to autograd's device thread) against loss.backward():
    the same losses, parameters and cache state after twelve iterations, bit for bit."""
    from hiscache import backward_on_this_thread
    la, _, ma, ca = _train(kind, 12, lambda loss: loss.backward())
    lb, _, mb, cb = _train(kind, 12, backward_on_this_thread)
    assert la == lb
    for (na, pa), (nb, pb) in zip(ma.named_parameters(), mb.named_parameters()):
        assert na == nb and torch.equal(pa, pb), na
    assert int(ca.header) == int(cb.header) and torch.equal(ca.table[: int(ca.header)], cb.table[: int(cb.header)])


def _train(kind, iters, backward):
    from hiscache import (HistoryRGCN, HistorySAGE, NeighborSampler, PinnedFeatureStore, RingHistoryCache, make_config,
                          prefer_low_latency_gemm)
    prefer_low_latency_gemm()
    N, Fin, H, C = 19_998, 32, 64, 6
    L = 3 if kind == "sage" else 2
    fanout = [6, 5, 4][:L]
    rng = np.random.default_rng(17)
    torch.manual_seed(17)
    # classes with their own feature mean, and neighbours mostly of a node's own class: the label can be read
    # from the node's features (SAGE's root term) and from its neighbourhood (the relational layer has no root term)
    labels = np.arange(N) % C
    deg = 8
    same = rng.random((N, deg)) < 0.9
    nb_class = np.where(same, labels[:, None], rng.integers(0, C, size=(N, deg)))
    indices = (rng.integers(0, N // C, size=(N, deg)) * C + nb_class).astype(np.int64).reshape(-1)
    indptr = np.arange(N + 1, dtype=np.int64) * deg
    centres = 1.5 * rng.standard_normal((C, Fin)).astype(np.float32)
    feats = (centres[labels] + rng.standard_normal((N, Fin), dtype=np.float32)).astype(np.float32)
    cache = RingHistoryCache(PinnedFeatureStore(torch.from_numpy(feats), device=DEV), N, Fin, H, capacity=N // 2,
                             num_layers=L, table_dtype=torch.float16, rate=0.3, age_limit=20, device=DEV)
    cfg = make_config(Fin, C, H, L, device=DEV, model_type=kind, num_rel=3)
    if kind == "sage":
        model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(DEV)
    else:
        model = HistoryRGCN(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache, num_rel=3).to(DEV)
    model.train()
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    # batches are sampled one ahead on the sampler's stream and come with the transposed view of their CSR
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=1, device=DEV, emit_view=True,
                              view_edges=kind == "rgcn")
    gen = torch.Generator(device=DEV).manual_seed(3)
    losses, hits = [], []
    pending = sampler.sample_async(torch.randperm(N, device=DEV, generator=gen)[:256])
    for it in range(1, iters + 1):
        batch = pending.get()
        pending = sampler.sample_async(torch.randperm(N, device=DEV, generator=gen)[:256])
        assert batch.view is not None and batch.view.num_edge == batch.idx.numel()
        if kind == "rgcn":
            batch.edge_type = (batch.idx % 3).contiguous()
        cache.lookup_and_load(batch, L)
        hits.append(float((cache.sub2embed != -1).float().mean()))
        loss = F.nll_loss(model(batch), batch.y)
        opt.zero_grad(set_to_none=True)
        backward(loss)
        opt.step()
        cache.update_history(batch, it)
        losses.append(float(loss.detach()))
    pending.get()
    return losses, hits, model, cache
