"""GPU parity of the host-side cache policy (HistoryCache, HistoryTable, the SAGE wiring) against the
torch-CPU restatement of the reference.  Index outputs, masks and cached-id sets bit-exact; embeddings
and gradients of the full model within 1e-5 relative of the same model evaluated on the CPU."""
import copy
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from helpers import layered_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_world(seed, N=3000, Fin=32, H=48, buffer_rows=400):
    from hiscache import HistoryCache, PinnedFeatureStore, make_config
    from oracle import host_model
    rng = np.random.default_rng(seed)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    hot = rng.permutation(N).astype(np.int64)
    lcm = np.lcm(Fin, H)
    buffer_floats = int(buffer_rows * lcm)
    cfg = make_config(Fin, 7, H, 3, method="grad", rate=0.6, staleness_thres=4, device=DEV)
    store = PinnedFeatureStore(feats, device=DEV)
    cache = HistoryCache(store, cfg, "history_uvm", total_num_node=N, buffer_bytes=buffer_floats * 4, hot_ids=hot)
    st = host_model.new_cache_state(N, Fin, H, buffer_floats, hot, feats)
    return rng, feats, cfg, cache, st


def batch_pair(rng, N, n_seed, fanout):
    from hiscache.synthetic import make_batch
    b = layered_batch(rng, N, n_seed, fanout)
    labels = rng.integers(0, 7, size=N)
    gpu = make_batch(b, labels, DEV)
    cpu = make_batch(b, labels, "cpu")
    return gpu, cpu


def assert_state_equal(cache, st):
    np.testing.assert_array_equal(cache.full2embed.cpu().numpy(), st.full2embed.numpy())
    np.testing.assert_array_equal(cache.embed2full.cpu().numpy(), st.embed2full.numpy())
    np.testing.assert_array_equal(cache.feat2full.cpu().numpy(), st.feat2full.numpy())
    assert cache.header == st.header


def test_fill_matches_model():
    rng, feats, cfg, cache, st = make_world(0)
    assert_state_equal(cache, st)
    n_feat = st.feat2full.numel()
    live = st.feat2full >= 0
    np.testing.assert_array_equal(cache.buffer.view(-1, st.Fin)[:n_feat][live.to(DEV)].cpu().numpy(),
                                  st.buffer.view(-1, st.Fin)[:n_feat][live].numpy())


def test_lookup_update_cycles_match_model():
    """Several iterations of lookup_and_load -> (synthetic gradients) -> update_history, including a
    staleness refresh, compared tensor by tensor with the CPU model."""
    from oracle import hc_oracle as orc
    from oracle import host_model
    rng, feats, cfg, cache, st = make_world(1)
    N, H = st.N, st.H
    want = dict(lookups=0, nodes=0, one_hop_nodes=0, embedding_hits=0, nodes_pruned=0, feature_hits=0, rows_loaded=0,
                rows_admitted=0)
    for it in range(1, 10):
        gpu, cpu = batch_pair(rng, N, 40, [6, 4, 3])
        cache.lookup_and_load(gpu, 3)
        ref = host_model.lookup_and_load(st, cpu, 3, feats)
        want["lookups"] += 1
        want["nodes"] += ref.sub2feat.numel()
        want["one_hop_nodes"] += ref.sub2embed.numel()
        want["embedding_hits"] += int((ref.sub2embed != -1).sum())
        want["nodes_pruned"] += int((~ref.used_masks[0]).sum())
        want["feature_hits"] += int((ref.sub2feat != -1).sum())
        want["rows_loaded"] += int(ref.load_mask.sum())
        np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), ref.sub2embed.numpy())
        np.testing.assert_array_equal(cache.sub2feat.cpu().numpy(), ref.sub2feat.numpy())
        for a, b in zip(cache.used_masks, ref.used_masks):
            np.testing.assert_array_equal(a.cpu().numpy(), b.numpy())
        np.testing.assert_array_equal(cache.load_mask.cpu().numpy(), ref.load_mask.numpy())
        np.testing.assert_array_equal(gpu.x.cpu().numpy(), ref.x.numpy())
        np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), ref.cached_embedding.numpy())
        # produced embeddings and their gradients for the 1-hop nodes
        n1 = int(cpu.num_node_in_layer[1])
        emb = rng.standard_normal((n1, H)).astype(np.float32)
        grad = (rng.standard_normal((n1, H)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)
        pe = torch.from_numpy(emb).to(DEV).requires_grad_(True)
        pe.grad = torch.from_numpy(grad).to(DEV)
        cache.produced_embedding = pe
        cache.update_history(gpu, it)
        score = torch.from_numpy(orc.row_scores(grad))
        mask, _ = host_model.update_history(st, cpu.sub_to_full, ref.sub2embed, torch.from_numpy(emb), score,
                                            0.6, 4, it)
        np.testing.assert_array_equal(cache.last_record_mask.cpu().numpy(), mask.numpy())
        want["rows_admitted"] += int(mask.sum())
        if it in (4, 9):
            # the counters of the lookups so far against the masks (the last admission has had no lookup behind it
            # yet and is added by stats() itself)
            got = cache.stats()
            assert {k: got[k] for k in want} == want
            assert got["embedding_hit_rate"] == want["embedding_hits"] / want["one_hop_nodes"]
            assert got["feature_hit_rate"] == want["feature_hits"] / want["nodes"]
            assert got["bytes_from_feature_store"] == want["rows_loaded"] * st.Fin * 4
        assert_state_equal(cache, st)
        n_emb = st.header
        np.testing.assert_array_equal(cache.buffer.view(-1, H)[:n_emb].cpu().numpy(),
                                      st.buffer.view(-1, H)[:n_emb].numpy())
        assert cache.produced_embedding is None and cache.overflow == 0
    s = cache.stats()
    assert s["embed_cached"] == int((st.full2embed[:N] != -1).sum())
    assert s["feat_cached"] == int((st.full2embed[N:2 * N] != -1).sum())


@pytest.mark.parametrize("speculative", [True, False])
def test_prefetched_features_give_the_same_batch(speculative):
    """``prefetch`` issued one batch ahead (before the previous batch's update changes the cache) leaves
    ``batch.x``, the slots, the masks and the cache state exactly as the unpipelined path does, for the
    buffer cache and the ring cache; reading the rows that the cache's state at that moment makes necessary
    (``speculative``) or every row."""
    from oracle import hc_oracle as orc
    from oracle import host_model
    from hiscache import PinnedFeatureStore, RingHistoryCache
    rng, feats, cfg, cache, st = make_world(5)
    N, H = st.N, st.H
    pairs = [batch_pair(rng, N, 40, [6, 4, 3]) for _ in range(6)]
    cache.prefetch(pairs[0][0], speculative=speculative)
    for it, (gpu, cpu) in enumerate(pairs, start=1):
        assert gpu.prefetched_x is not None
        cache.lookup_and_load(gpu, 3)
        assert gpu.prefetched_x is None                      # consumed
        if it < len(pairs):
            cache.prefetch(pairs[it][0], speculative=speculative)   # next batch, before this batch's update
        ref = host_model.lookup_and_load(st, cpu, 3, feats)
        np.testing.assert_array_equal(gpu.x.cpu().numpy(), ref.x.numpy())
        np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), ref.sub2embed.numpy())
        np.testing.assert_array_equal(cache.load_mask.cpu().numpy(), ref.load_mask.numpy())
        np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), ref.cached_embedding.numpy())
        n1 = int(cpu.num_node_in_layer[1])
        emb = rng.standard_normal((n1, H)).astype(np.float32)
        grad = (rng.standard_normal((n1, H)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)
        pe = torch.from_numpy(emb).to(DEV).requires_grad_(True)
        pe.grad = torch.from_numpy(grad).to(DEV)
        cache.produced_embedding = pe
        cache.update_history(gpu, it)
        host_model.update_history(st, cpu.sub_to_full, ref.sub2embed, torch.from_numpy(emb),
                                  torch.from_numpy(orc.row_scores(grad)), 0.6, 4, it)
        assert_state_equal(cache, st)
    # a handle made for other ids is ignored
    gpu, cpu = batch_pair(rng, N, 30, [5, 3, 2])
    cache.prefetch(gpu, speculative=speculative)
    gpu.sub_to_full = gpu.sub_to_full.clone()
    cache.lookup_and_load(gpu, 3)
    np.testing.assert_array_equal(gpu.x.cpu().numpy(), host_model.lookup_and_load(st, cpu, 3, feats).x.numpy())

    # the store's side-stream read of a masked subset equals the plain one
    store = cache.uvm
    m = torch.from_numpy(rng.random(gpu.sub_to_full.numel()) < 0.5).to(DEV)
    rows, done = store.masked_get_async(gpu.sub_to_full, m)
    store.join(done)
    np.testing.assert_array_equal(rows.cpu().numpy(), store.masked_get(gpu.sub_to_full, m).cpu().numpy())

    # ring cache: two caches in the same state, one pipelined
    from hiscache.synthetic import make_batch
    ring = [RingHistoryCache(PinnedFeatureStore(feats, device=DEV), N, st.Fin, 64, capacity=500, num_layers=3,
                             table_dtype=torch.float16, thres=0.05, age_limit=3, device=DEV) for _ in range(2)]
    bs = [layered_batch(rng, N, 40, [6, 4, 3]) for _ in range(5)]
    mk = lambda b: make_batch(b, np.zeros(N, np.int64), DEV)
    nxt = mk(bs[0])
    ring[1].prefetch(nxt, speculative=speculative)
    for it, b in enumerate(bs, start=1):
        plain, piped = mk(b), nxt
        ring[0].lookup_and_load(plain, 3)
        ring[1].lookup_and_load(piped, 3)
        if it < len(bs):
            nxt = mk(bs[it])
            ring[1].prefetch(nxt, speculative=speculative)
        np.testing.assert_array_equal(piped.x.cpu().numpy(), plain.x.cpu().numpy())
        np.testing.assert_array_equal(ring[1].cached_embedding.cpu().numpy(), ring[0].cached_embedding.cpu().numpy())
        n1 = int(b["num_node_in_layer"][1])
        emb = torch.from_numpy(rng.standard_normal((n1, 64)).astype(np.float32)).to(DEV)
        grad = torch.from_numpy((rng.standard_normal((n1, 64)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)).to(DEV)
        for c, bb in zip(ring, (plain, piped)):
            pe = emb.clone().requires_grad_(True)
            pe.grad = grad.clone()
            c.produced_embedding = pe
            c.update_history(bb, it)
        np.testing.assert_array_equal(ring[1].full2slot.cpu().numpy(), ring[0].full2slot.cpu().numpy())
    assert ring[0].header > 0


@pytest.mark.parametrize("src_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float16, torch.float16),
                                                 (torch.float16, torch.float32)])
def test_fixup_rows_turns_a_guessed_gather_into_the_exact_one(src_dtype, out_dtype):
    """hc_fixup_rows: rows read under a guessed mask become the rows of the exact mask -- missing rows are
    read (from pinned host memory, zero-copy), surplus rows cleared, the others not touched."""
    import hiscache_backend as be
    rng = np.random.default_rng(21)
    n_rows, F, n = 5000, 96, 3000
    table = torch.from_numpy(rng.standard_normal((n_rows, F)).astype(np.float32)).to(src_dtype).pin_memory()
    ids = torch.from_numpy(rng.integers(-5, n_rows, size=n)).to(DEV)           # a few negative ids: from the end
    have = torch.from_numpy(rng.random(n) < 0.6).to(DEV)
    need = torch.from_numpy(rng.random(n) < 0.6).to(DEV)
    out = be.gather_rows(table, ids, mask=have, out_dtype=out_dtype)
    same = (have == need)
    marker = out[same].clone()
    be.fixup_rows(table, ids, need, have, out)
    want = be.gather_rows(table, ids, mask=need, out_dtype=out_dtype)
    assert torch.equal(out, want)
    assert torch.equal(out[same], marker)
    assert int((need & ~have).sum()) > 100 and int((have & ~need).sum()) > 100
    # nothing to fix: the call leaves the rows alone
    before = out.clone()
    be.fixup_rows(table, ids, need, need, out)
    assert torch.equal(out, before)


def test_gather_rows_on_a_named_stream():
    """gather_rows(stream=side) enqueues on that stream without switching torch's current one: the rows are
    those of the call on the current stream once the streams have been ordered."""
    import hiscache_backend as be
    rng = np.random.default_rng(22)
    table = torch.from_numpy(rng.standard_normal((4000, 64)).astype(np.float32)).pin_memory()
    ids = torch.from_numpy(rng.integers(0, 4000, size=2500)).to(DEV)
    mask = torch.from_numpy(rng.random(2500) < 0.7).to(DEV)
    want = be.gather_rows(table, ids, mask=mask)
    side = torch.cuda.Stream()
    cur = torch.cuda.current_stream()
    side.wait_stream(cur)
    got = be.gather_rows(table, ids, mask=mask, stream=side)
    got.record_stream(side)
    assert torch.cuda.current_stream() == cur
    cur.wait_stream(side)
    assert torch.equal(got, want)


@pytest.mark.parametrize("prefetch_cus", [0, 16])
def test_speculative_prefetch_is_fixed_up_at_the_lookup(prefetch_cus):
    """The ring cache's read-ahead runs under the masks of the cache state at that moment; entries that are
    admitted, or whose slot is given up, between the read-ahead and the lookup change which rows are needed.
    ``batch.x`` still equals the unpipelined result, and the test makes sure rows moved in both directions.
    With ``prefetch_cus`` the read runs on a stream kept to that many compute units."""
    from hiscache import PinnedFeatureStore, RingHistoryCache
    from hiscache.synthetic import make_batch
    rng = np.random.default_rng(33)
    N, Fin, H = 4000, 32, 64
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    caches = [RingHistoryCache(PinnedFeatureStore(feats, device=DEV, prefetch_cus=cus), N, Fin, H, capacity=2000,
                               num_layers=3, table_dtype=torch.float16, thres=0.05, age_limit=1000, device=DEV)
              for cus in (0, prefetch_cus)]
    b = layered_batch(rng, N, 60, [6, 5, 4])
    n1 = int(b["num_node_in_layer"][1])
    hop1 = b["sub_to_full"][:n1]
    first = torch.from_numpy(hop1[: n1 // 3].copy()).to(DEV)        # cached when the read-ahead starts
    later = torch.from_numpy(hop1[n1 // 3: 2 * n1 // 3].copy()).to(DEV)  # admitted in between
    rows = torch.from_numpy(rng.standard_normal((n1, H)).astype(np.float32)).to(DEV)
    for c in caches:
        c.preload(first, rows[: first.numel()])
    plain, piped = (make_batch(b, np.zeros(N, np.int64), DEV) for _ in range(2))
    compute = torch.cuda.Stream()                                  # the read-ahead overlaps a non-default stream
    compute.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(compute):
        caches[1].prefetch(piped)
        have = piped.prefetched_x.mask.clone()
        for c in caches:                                            # the cache changes before the lookup
            c.preload(later, rows[first.numel(): first.numel() + later.numel()])
            c.full2slot[first[::2]] = -1                            # every other early entry gives up its slot
        caches[0].lookup_and_load(plain, 3)
        caches[1].lookup_and_load(piped, 3)
        need = caches[1].used_masks[0]
        assert int((need & ~have).sum()) > 0 and int((have & ~need).sum()) > 0
        assert torch.equal(piped.x, plain.x)
        assert torch.equal(caches[1].sub2embed, caches[0].sub2embed)
        ref = feats.to(DEV)[piped.sub_to_full] * need[:, None]
        assert torch.equal(piped.x, ref)
    torch.cuda.current_stream().wait_stream(compute)
    torch.cuda.synchronize()


def test_update_history_overflow_is_counted():
    from oracle import hc_oracle as orc
    from oracle import host_model
    rng, feats, cfg, cache, st = make_world(2, buffer_rows=2)       # room for very few embedding rows
    N, H = st.N, st.H
    cap = st.embed2full.numel()
    gpu, cpu = batch_pair(rng, N, 60, [8, 4, 2])
    cache.lookup_and_load(gpu, 3)
    ref = host_model.lookup_and_load(st, cpu, 3, feats)
    n1 = int(cpu.num_node_in_layer[1])
    emb = rng.standard_normal((n1, H)).astype(np.float32)
    grad = rng.standard_normal((n1, H)).astype(np.float32)
    pe = torch.from_numpy(emb).to(DEV).requires_grad_(True)
    pe.grad = torch.from_numpy(grad).to(DEV)
    cache.produced_embedding = pe
    cache.update_history(gpu, 1)
    mask, _ = host_model.update_history(st, cpu.sub_to_full, ref.sub2embed, torch.from_numpy(emb),
                                        torch.from_numpy(orc.row_scores(grad)), 0.6, 4, 1)
    assert int(mask.sum()) > cap
    assert cache.header == cap == st.header and cache.overflow == int(mask.sum()) - cap
    assert_state_equal(cache, st)


def test_feature_cache_only_and_no_cache_modes():
    from hiscache import HistoryCache, PinnedFeatureStore, make_config
    rng, feats, cfg, cache, st = make_world(3)
    gpu, cpu = batch_pair(rng, st.N, 30, [5, 3, 2])
    cache.lookup_and_load(gpu, 3, feature_cache_only=True)
    np.testing.assert_array_equal(gpu.x.cpu().numpy(), feats[cpu.sub_to_full].numpy())
    plain = HistoryCache(PinnedFeatureStore(feats, device=DEV), cfg, "uvm", total_num_node=st.N)
    plain.lookup_and_load(gpu, 3)
    np.testing.assert_array_equal(gpu.x.cpu().numpy(), feats[cpu.sub_to_full].numpy())
    assert (plain.sub2embed == -1).all() and plain.cached_embedding.numel() == 0
    plain.update_history(gpu, 1)            # a no-op without a history buffer


class CpuSage(torch.nn.Module):
    """The same network evaluated with dense CPU operators (mean aggregation by index_add)."""

    def __init__(self, model):
        super().__init__()
        table, model.table = model.table, None          # the cache (streams, device buffers) is not copied
        try:
            self.m = copy.deepcopy(model).cpu()
        finally:
            model.table = table

    def forward(self, batch, x, sub2embed, cached_embedding):
        from oracle import torch_cpu_path as tp
        m = self.m
        L = m.num_layers
        his_out = None
        for i, conv in enumerate(m.convs):
            n = int(batch.num_node_in_layer[L - 1 - i])
            if m.training and i == L - 2:
                # differentiable statement of the history layer
                agg = mean_rows(x, batch.ptr, batch.idx, n)
                hit = (sub2embed != -1)[:, None]
                agg = torch.where(hit, cached_embedding, agg)
                if not agg.requires_grad:               # history layer on raw features (2-layer models)
                    agg.requires_grad_(True)
                agg.retain_grad()
                his_out = agg
            else:
                agg = mean_rows(x, batch.ptr, batch.idx, n)
            x = conv.lin_l(agg) + conv.lin_r(x[:n])
            if i < L - 1:
                x = m.bns[i](x)
                x = torch.relu(x)
        return x.log_softmax(dim=-1), his_out


def mean_rows(x, ptr, idx, n):
    deg = (ptr[1:n + 1] - ptr[:n])
    dst = torch.repeat_interleave(torch.arange(n), deg)
    out = torch.zeros(n, x.shape[1], dtype=x.dtype)
    out = out.index_add(0, dst, x[idx[: int(ptr[n])]])
    return out / deg.clamp(min=1).to(x.dtype)[:, None]


def test_sage_training_iteration_matches_cpu():
    """lookup_and_load -> HistorySAGE forward -> loss.backward -> update_history on the GPU, against the
    same network on the CPU: logits, the gradient reaching the produced embedding, parameter gradients
    (1e-5 relative, fp32) and the admitted id set (exact, thresholds kept away from knife edges)."""
    from hiscache import get_model
    from oracle import hc_oracle as orc
    from oracle import host_model
    torch.manual_seed(0)
    rng, feats, cfg, cache, st = make_world(4, N=4000, Fin=64, H=128, buffer_rows=300)
    N, H = st.N, st.H
    model = get_model(cfg, cache).to(DEV)
    model.train()
    cpu_model = CpuSage(model)
    cpu_model.m.train()
    for it in range(1, 4):
        gpu, cpu = batch_pair(rng, N, 50, [6, 4, 3])
        cache.lookup_and_load(gpu, 3)
        ref = host_model.lookup_and_load(st, cpu, 3, feats)
        out = model(gpu)
        loss = torch.nn.functional.nll_loss(out, gpu.y)
        model.zero_grad()
        loss.backward()
        out_c, his_c = cpu_model(cpu, ref.x, ref.sub2embed, ref.cached_embedding)
        loss_c = torch.nn.functional.nll_loss(out_c, cpu.y)
        cpu_model.m.zero_grad()
        loss_c.backward()
        np.testing.assert_allclose(out.detach().cpu().numpy(), out_c.detach().numpy(), rtol=1e-4, atol=1e-5)
        pe = cache.produced_embedding
        assert pe is not None and pe.grad is not None
        np.testing.assert_allclose(pe.detach().cpu().numpy(), his_c.detach().numpy(), rtol=1e-5, atol=1e-6)
        scale = float(his_c.grad.abs().max())
        np.testing.assert_allclose(pe.grad.cpu().numpy(), his_c.grad.numpy(), rtol=1e-3, atol=1e-5 * scale)
        # biases in front of a batch norm have a mathematically zero gradient (pure rounding noise), so
        # the absolute floor is taken from the largest parameter gradient of the network
        gscale = max(float(q.grad.abs().max()) for q in cpu_model.m.parameters() if q.grad is not None)
        for (n_, p), (_, q) in zip(model.named_parameters(), cpu_model.m.named_parameters()):
            if p.grad is None:
                continue
            np.testing.assert_allclose(p.grad.cpu().numpy(), q.grad.numpy(), rtol=1e-3, atol=2e-5 * gscale,
                                       err_msg=n_)
        # admission on the GPU gradient itself, mirrored on the CPU model state
        grad_gpu = pe.grad.cpu().numpy()
        emb_gpu = pe.detach().cpu().numpy()
        cache.update_history(gpu, it)
        score = torch.from_numpy(orc.row_scores(grad_gpu))
        mask, _ = host_model.update_history(st, cpu.sub_to_full, ref.sub2embed, torch.from_numpy(emb_gpu), score,
                                            0.6, 4, it)
        np.testing.assert_array_equal(cache.last_record_mask.cpu().numpy(), mask.numpy())
        assert_state_equal(cache, st)
    model.eval()
    gpu, cpu = batch_pair(rng, N, 20, [4, 3, 2])
    cache.lookup_and_load(gpu, 3, feature_cache_only=True)
    with torch.no_grad():
        ev = model(gpu)
    assert ev.shape == (20, 7) and torch.isfinite(ev).all()


def test_fused_sage_layer_equals_the_operator_by_operator_spelling():
    """MySageConvHistory as one autograd node (aggregation, both linear maps, the root term's gradient
    accumulated into the aggregation's input gradient) against the same layer spelled operator by
    operator: identical aggregation output and produced-embedding gradient, outputs and parameter
    gradients to fp32 GEMM rounding."""
    from hiscache import MySageConvHistory
    from helpers import random_csr, random_hmap
    rng = np.random.default_rng(31)
    torch.manual_seed(31)
    R, N, Fin, H = 700, 1500, 128, 64
    ptr, idx = random_csr(rng, R, N, 9, hub=300)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    hmap = t(random_hmap(rng, R, 0.3))
    hbuf = t(rng.standard_normal((R, Fin)).astype(np.float32))
    g = t(rng.standard_normal((R, H)).astype(np.float32))
    conv = MySageConvHistory(Fin, H, need_grad=True).to(DEV)
    conv.train()
    res = {}
    for fused in (True, False):
        conv.fused = fused
        conv.zero_grad()
        x = t(rng.standard_normal((N, Fin)).astype(np.float32) * 0 + 1).requires_grad_(True)
        x.data.copy_(t(np.random.default_rng(5).standard_normal((N, Fin)).astype(np.float32)))
        out, his = conv(x, t(ptr), t(idx), hmap, hbuf, Fin, R, int(ptr[R]))
        out.backward(g)
        res[fused] = (out.detach(), his.detach(), his.grad.clone(), x.grad.clone(), conv.lin_l.weight.grad.clone(),
                      conv.lin_l.bias.grad.clone(), conv.lin_r.weight.grad.clone())
    a, b = res[True], res[False]
    assert torch.equal(a[1], b[1])                                   # aggregation output, bit for bit
    for i, name in ((0, "out"), (2, "his.grad"), (3, "x.grad"), (4, "lin_l.weight.grad"), (5, "lin_l.bias.grad"),
                    (6, "lin_r.weight.grad")):
        scale = float(b[i].abs().max())
        np.testing.assert_allclose(a[i].cpu().numpy(), b[i].cpu().numpy(), rtol=1e-4, atol=1e-5 * scale, err_msg=name)
    # without history and without a gradient sink the fused layer still returns the aggregation
    conv.fused = True
    none = torch.empty(0, device=DEV)
    out2, his2 = conv(t(rng.standard_normal((N, Fin)).astype(np.float32)), t(ptr), t(idx), none, none, 0, R)
    assert his2.grad is None and tuple(out2.shape) == (R, H)


def test_history_table_record_and_evict():
    from hiscache import HistoryTable, make_config
    from oracle import hc_oracle as orc
    from oracle import host_model
    rng = np.random.default_rng(5)
    N, Fin, H = 2000, 16, 24
    cfg = make_config(Fin, 5, H, 3, method="grad", rate=0.7, staleness_thres=3, device=DEV, model_type="SAGE",
                      buffer_size=150)
    table = HistoryTable(cfg, total_num_node=N)
    assert table.num_layers == 2 and table.history_size_layered == [Fin, H]
    ref = [dict(buf=np.zeros((150, w), np.float32), h2f=np.full(150, -1, np.int64), f2h=np.full(N, -1, np.int64),
                checkin=np.full(150, -1, np.int64), header=np.zeros(1, np.int64)) for w in (Fin, H)]
    for it in range(1, 7):
        b = layered_batch(rng, N, 25, [5, 4, 3])
        nnl = b["num_node_in_layer"]
        from hiscache.synthetic import make_batch
        batch = make_batch(b, rng.integers(0, 5, size=N), DEV)
        batch.x = torch.zeros((int(nnl[-1]), Fin), device=DEV)
        table.lookup(batch.sub_to_full, nnl)
        used = orc.count_history_reconstruct(b["ptr"], b["idx"], None, int(nnl[-1]), 25, 3)
        used_dev = [torch.from_numpy(u).to(DEV) for u in used]
        table.history_out = []
        outs = []
        for layer_id, w in enumerate((Fin, H)):
            n = int(nnl[3 - 1 - layer_id])
            his = torch.from_numpy(rng.standard_normal((n, w)).astype(np.float32)).to(DEV).requires_grad_(True)
            his.grad = torch.from_numpy((rng.standard_normal((n, w)) * np.exp(rng.normal(-3, 1, size=(n, 1)))
                                         ).astype(np.float32)).to(DEV)
            table.history_out.append(his)
            outs.append(his)
            s2h = table.sub_to_history[layer_id].cpu().numpy()
            expect = ref[layer_id]["f2h"][b["sub_to_full"][:n]].copy()
            expect[:25] = -1
            np.testing.assert_array_equal(s2h, expect)
            # compact ids and compact buffer
            comp = table.sub_to_history_layered[layer_id].cpu().numpy()
            hit = expect != -1
            np.testing.assert_array_equal(comp[hit], np.arange(hit.sum()))
            assert (comp[~hit] == -1).all()
            np.testing.assert_array_equal(table.tmp_history_buffer_layered[layer_id].detach().cpu().numpy(),
                                          ref[layer_id]["buf"][expect[hit]])
        table.record_history(batch.sub_to_full, batch, it, used_dev)
        for layer_id, w in enumerate((Fin, H)):
            n = int(nnl[3 - 1 - layer_id])
            r = ref[layer_id]
            score = orc.row_scores(outs[layer_id].grad.cpu().numpy(), orc.NORM_L1)
            thres = host_model.quantile_threshold(score, 0.7)
            s2h = r["f2h"][b["sub_to_full"][:n]].copy()
            s2h[:25] = -1
            orc.record_history(outs[layer_id].detach().cpu().numpy(), r["buf"], used[layer_id + 1][:n],
                               b["sub_to_full"], s2h, r["h2f"], r["f2h"], r["header"], score, thres, r["checkin"], it)
            np.testing.assert_array_equal(table.history_to_full_layered[layer_id].cpu().numpy(), r["h2f"])
            np.testing.assert_array_equal(table.full_to_history_layered[layer_id].cpu().numpy(), r["f2h"])
            np.testing.assert_array_equal(table.checkin_iter[layer_id].cpu().numpy(), r["checkin"])
            np.testing.assert_array_equal(table.cuda_header_layered[layer_id].cpu().numpy(), r["header"])
            live = r["h2f"] != -1
            np.testing.assert_array_equal(table.history_buffer_layered[layer_id].cpu().numpy()[live], r["buf"][live])
        if it == 5:
            # gradient eviction + staleness eviction (HistoryTable.evict_by_both)
            table.evict_by_both(batch, it, 3)
            for layer_id in range(2):
                n = int(nnl[3 - 1 - layer_id])
                r = ref[layer_id]
                score = torch.from_numpy(orc.row_scores(outs[layer_id].grad.cpu().numpy(), orc.NORM_L1))
                s2h = table.sub_to_history[layer_id][:n].cpu()
                c, h, f = (torch.from_numpy(r[k]) for k in ("checkin", "h2f", "f2h"))
                host_model.evict_by_both(c, h, f, s2h, score, 0.7, it, 3)
                np.testing.assert_array_equal(table.history_to_full_layered[layer_id].cpu().numpy(), r["h2f"])
                np.testing.assert_array_equal(table.full_to_history_layered[layer_id].cpu().numpy(), r["f2h"])
                np.testing.assert_array_equal(table.checkin_iter[layer_id].cpu().numpy(), r["checkin"])
        elif it % 2 == 0:
            table.evict_by_staleness(it, 3)
            for layer_id in range(2):
                r = ref[layer_id]
                c, h, f = (torch.from_numpy(r[k]) for k in ("checkin", "h2f", "f2h"))
                host_model.evict_by_staleness(c, h, f, it, 3)
                np.testing.assert_array_equal(table.history_to_full_layered[layer_id].cpu().numpy(), r["h2f"])
                np.testing.assert_array_equal(table.full_to_history_layered[layer_id].cpu().numpy(), r["f2h"])
    assert sum(table.show()) > 0


def test_ring_cache_cycles_match_oracle():
    """RingHistoryCache (fp16 ring table, fused admission with staleness ages, fixed threshold and
    quantile threshold) against the CPU oracle's grad_check over several iterations."""
    from hiscache import PinnedFeatureStore, RingHistoryCache
    from oracle import hc_oracle as orc
    from oracle import host_model
    from hiscache.synthetic import make_batch
    rng = np.random.default_rng(6)
    N, Fin, H, cap = 3000, 32, 64, 500
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    for fixed in (True, False):
        cache = RingHistoryCache(PinnedFeatureStore(feats, device=DEV), N, Fin, H, capacity=cap, num_layers=3,
                                 table_dtype=torch.float16, thres=0.05 if fixed else None, rate=0.6, age_limit=3,
                                 device=DEV)
        ref = dict(table=np.zeros((cap, H), np.uint16), f2s=np.full(N, -1, np.int64), s2f=np.full(cap, -1, np.int64),
                   checkin=np.full(cap, -1, np.int64), header=np.zeros(1, np.int64))
        n_stale = 0
        stat = dict(admitted=0, hits=0, loaded=0, nodes=0)
        for it in range(1, 9):
            b = layered_batch(rng, N, 40, [6, 4, 3])
            batch = make_batch(b, rng.integers(0, 5, size=N), DEV)
            cache.lookup_and_load(batch, 3)
            n1 = int(b["num_node_in_layer"][1])
            nodes = b["sub_to_full"][:n1]
            # entries that are 3 iterations old count as absent at lookup (the cache's counter equals `it`)
            tab32 = ref["table"].view(np.float16).astype(np.float32)
            slot, rows = host_model.ring_lookup(ref["f2s"], ref["checkin"], nodes, it, 3, tab32)
            n_stale += int(((ref["f2s"][nodes] != -1) & (slot == -1)).sum())
            np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), slot)
            np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), rows)
            used = orc.count_history_reconstruct(b["ptr"], b["idx"], slot, len(b["sub_to_full"]), 40, 3)
            np.testing.assert_array_equal(cache.used_masks[0].cpu().numpy(), used[0])
            stat["hits"] += int((slot != -1).sum())
            stat["loaded"] += int(used[0].sum())
            stat["nodes"] += len(b["sub_to_full"])
            x_ref = feats[torch.from_numpy(b["sub_to_full"])].numpy() * used[0][:, None]
            np.testing.assert_array_equal(batch.x.cpu().numpy(), x_ref)
            emb = rng.standard_normal((n1, H)).astype(np.float32)
            grad = (rng.standard_normal((n1, H)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)
            pe = torch.from_numpy(emb).to(DEV).requires_grad_(True)
            pe.grad = torch.from_numpy(grad).to(DEV)
            cache.produced_embedding = pe
            cache.update_history(batch, it)
            score = orc.row_scores(grad)
            thres = 0.05 if fixed else float(host_model.quantile_threshold(score, 0.6))
            rmask, _, _ = orc.grad_check(grad, emb, slot, None, None, nodes, thres, 0, orc.NORM_L2, orc.CMP_LT,
                                         ref["table"], orc.DT_F16, ref["f2s"], ref["s2f"], ref["checkin"],
                                         ref["header"], it)
            np.testing.assert_array_equal(cache.last_record_mask.cpu().numpy(), rmask)
            stat["admitted"] += int(rmask.sum())
            np.testing.assert_array_equal(cache.full2slot.cpu().numpy(), ref["f2s"])
            np.testing.assert_array_equal(cache.slot2full.cpu().numpy(), ref["s2f"])
            np.testing.assert_array_equal(cache.checkin.cpu().numpy(), ref["checkin"])
            assert cache.header == int(ref["header"][0])
            live = ref["s2f"] != -1
            np.testing.assert_array_equal(cache.table.view(torch.int16).cpu().numpy().view(np.uint16)[live],
                                          ref["table"][live])
        assert (ref["s2f"] != -1).sum() > 0 and n_stale > 0
        got = cache.stats()
        assert got["lookups"] == 8 and got["embed_cached"] == int((ref["f2s"] != -1).sum())
        assert got["rows_admitted"] == stat["admitted"] and got["embedding_hits"] == stat["hits"]
        assert got["rows_loaded"] == stat["loaded"] and got["nodes_pruned"] == stat["nodes"] - stat["loaded"]
        assert got["bytes_from_feature_store"] == stat["loaded"] * Fin * 4


def test_ring_cache_refreshes_stale_entries_with_recomputed_values():
    """An entry that reaches the age limit is reported absent at lookup, so the model recomputes the
    row and the admission stores the NEW value in a new slot; an entry below the limit is served from
    the table and is not re-admitted.  Driven with the model's own history-layer output."""
    from hiscache import HistorySAGE, PinnedFeatureStore, RingHistoryCache, make_config
    from hiscache.synthetic import make_batch
    rng = np.random.default_rng(66)
    torch.manual_seed(66)
    N, Fin, H, C, L = 2000, 64, 64, 4, 3       # 3 layers: the history layer's input depends on weights
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    cache = RingHistoryCache(PinnedFeatureStore(feats, device=DEV), N, Fin, H, capacity=4000, num_layers=L,
                             table_dtype=torch.float32, thres=1e9, age_limit=2, device=DEV)   # every row passes
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device=DEV), cache).to(DEV)
    model.train()
    opt = torch.optim.SGD(model.parameters(), lr=0.5)
    b = layered_batch(rng, N, 30, [5, 4, 3])
    batch = make_batch(b, rng.integers(0, C, size=N), DEV)
    n1 = int(b["num_node_in_layer"][1])
    stored, slots = [], []
    for it in range(1, 5):
        cache.lookup_and_load(batch, L)
        hit = (cache.sub2embed != -1).cpu().numpy()
        out = model(batch)
        loss = torch.nn.functional.nll_loss(out, batch.y)
        opt.zero_grad()
        loss.backward()
        opt.step()
        pe = cache.produced_embedding.detach().clone()
        cache.update_history(batch, it)
        mask = cache.last_record_mask.cpu().numpy()
        f2s = cache.full2slot[batch.sub_to_full[:n1]].cpu().numpy()
        tab = cache.table[torch.from_numpy(np.maximum(f2s, 0)).to(DEV)].cpu().numpy()
        if it == 1:                       # nothing cached: everything is computed and admitted
            assert not hit.any() and mask.all()
        elif it == 2:                     # age 1 < 2: served from the table, nothing re-admitted
            assert hit.all() and not mask.any()
            np.testing.assert_array_equal(pe.cpu().numpy(), stored[0])
            np.testing.assert_array_equal(f2s, slots[0])
        elif it == 3:                     # age 2: stale -> recomputed with the trained weights, re-admitted
            assert not hit.any() and mask.all()
            assert (f2s != slots[0]).all()
            assert np.abs(pe.cpu().numpy() - stored[0]).max() > 1e-4     # the fresh value differs
        np.testing.assert_array_equal(tab, pe.cpu().numpy() if mask.all() else stored[-1])
        stored.append(tab.copy())
        slots.append(f2s.copy())


def test_input_layer_backward_is_skipped_but_history_grad_is_kept():
    import hiscache_backend as be
    from helpers import random_csr, random_hmap
    from oracle import hc_oracle as orc
    rng = np.random.default_rng(7)
    R, N, F = 80, 60, 128
    ptr, idx = random_csr(rng, R, N, 6)
    hmap = random_hmap(rng, R, 0.4)
    x = torch.from_numpy(rng.standard_normal((N, F)).astype(np.float32)).to(DEV)        # raw features: no grad
    hb = torch.from_numpy(rng.standard_normal((R, F)).astype(np.float32)).to(DEV).requires_grad_(True)
    g = rng.standard_normal((R, F)).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(DEV)
    out = be.aggr_forward_history(x, t(ptr), t(idx), t(hmap), hb, F, R)
    out.backward(t(g))
    assert x.grad is None
    np.testing.assert_array_equal(hb.grad.cpu().numpy(), orc.bwd_mean_row(ptr, idx, g, hmap, N, (R, F))[1])


def rgcn_layer_cpu(x, W, ptr, idx, rel, used, n, hit=None, hbuf=None):
    """sum_j x[src_j] @ W[rel_j] / deg over the first n rows, unused sources dropped, in fp64."""
    deg = (ptr[1:n + 1] - ptr[:n])
    E = int(ptr[n])
    dst = torch.repeat_interleave(torch.arange(n), deg)
    src = idx[:E]
    msg = torch.einsum("ef,efh->eh", x[src].double(), W.double()[rel[:E]])
    if used is not None:
        msg = msg * used[src][:, None]
    out = torch.zeros(n, W.shape[2], dtype=torch.float64).index_add(0, dst, msg)
    out = out / deg.clamp(min=1)[:, None]
    if hit is not None:
        out = torch.where(hit[:, None], hbuf.double(), out)
    return out


@pytest.mark.parametrize("feat_dtype", [torch.float32, torch.float16])
def test_rgcn_typed_aggregation_matches_dense_cpu(feat_dtype):
    """HistoryRGCN (typed gather-reduce over (row, relation) groups + one GEMM) against a dense fp64
    statement of sum_j x[src_j] @ W[rel_j] / deg with history substitution; gradients too."""
    from hiscache import HistoryRGCN, PinnedFeatureStore, RingHistoryCache, make_config
    from hiscache.synthetic import make_batch
    rng = np.random.default_rng(8)
    torch.manual_seed(1)
    N, Fin, H, C, K, L = 3000, 128, 64, 6, 5, 2
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32)).to(feat_dtype)
    cache = RingHistoryCache(PinnedFeatureStore(feats, device=DEV), N, Fin, H, capacity=800, num_layers=L,
                             table_dtype=torch.float32, thres=0.5, device=DEV)
    pre = torch.from_numpy(rng.choice(N, size=700, replace=False)).to(DEV)
    cache.preload(pre, torch.randn(700, H, device=DEV))
    cfg = make_config(Fin, C, H, L, device=DEV, model_type="rgcn", num_rel=K)
    model = HistoryRGCN(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache, num_rel=K).to(DEV)
    model.train()
    b = layered_batch(rng, N, 40, [6, 4])
    batch = make_batch(b, rng.integers(0, C, size=N), DEV)
    batch.edge_type = torch.from_numpy(rng.integers(0, K, size=len(b["idx"]))).to(DEV)
    cache.lookup_and_load(batch, L)
    out = model(batch)
    loss = torch.nn.functional.nll_loss(out, batch.y)
    loss.backward()
    # the same network in fp64 on the CPU
    nnl = b["num_node_in_layer"]
    ptr, idx = torch.from_numpy(b["ptr"]), torch.from_numpy(b["idx"])
    rel = batch.edge_type.cpu()
    used = [m.cpu() for m in cache.used_masks]
    x0 = batch.x.cpu()
    W0 = model.convs[0].linear.detach().cpu().double().requires_grad_(True)
    W1 = model.convs[1].linear.detach().cpu().double().requires_grad_(True)
    n1, n0 = int(nnl[1]), int(nnl[0])
    hit = cache.sub2embed.cpu() != -1
    assert hit.any() and (~hit).any() and (~used[0]).any()
    h1 = rgcn_layer_cpu(x0, W0, ptr, idx, rel, used[0].double(), n1, hit, cache.cached_embedding.cpu())
    h1.retain_grad()
    bn = model.bns[0]
    mu, var = h1.mean(0), h1.var(0, unbiased=False)
    z = (h1 - mu) / torch.sqrt(var + bn.eps) * bn.weight.detach().cpu().double() + bn.bias.detach().cpu().double()
    z = torch.relu(z)
    o = rgcn_layer_cpu(z, W1, ptr, idx, rel, used[-2].double(), n0).log_softmax(dim=-1)
    loss_c = torch.nn.functional.nll_loss(o, batch.y.cpu())
    loss_c.backward()
    tol = 2e-3 if feat_dtype == torch.float16 else 2e-4
    np.testing.assert_allclose(out.detach().cpu().numpy(), o.detach().numpy(), rtol=tol, atol=tol)
    pe = cache.produced_embedding
    gs = float(h1.grad.abs().max())
    np.testing.assert_allclose(pe.grad.cpu().numpy(), h1.grad.numpy(), rtol=1e-2, atol=tol * gs)
    for got, ref in ((model.convs[0].linear.grad, W0.grad), (model.convs[1].linear.grad, W1.grad)):
        s = float(ref.abs().max())
        np.testing.assert_allclose(got.cpu().numpy(), ref.numpy(), rtol=1e-2, atol=tol * s)
    cache.update_history(batch, 1)
    assert cache.last_record_mask.shape[0] == n1


@pytest.mark.parametrize("feat_dtype", [torch.float32, torch.float16])
def test_fused_rgcn_layer_equals_the_operator_by_operator_spelling(feat_dtype):
    """_RgcnConvFunction (edge weights 1/deg, one node) against the spelling with group means rescaled by
    cnt/deg and torch's autograd: outputs, weight gradient, input gradient, gradient kept on the history
    layer's output; with and without history, at an inner size on either side of the split-GEMM switch."""
    from hiscache.history_model import MyRGCNConvHistory2
    from helpers import random_csr
    rng = np.random.default_rng(21)
    torch.manual_seed(4)
    for (R, N, Fin, H, K, use_hist, x_grad) in ((300, 900, 64, 32, 5, True, True), (700, 2000, 512, 64, 5, True, False),
                                                (41, 200, 448, 16, 5, False, True)):
        ptr, idx = random_csr(rng, R + 30, N, 9)
        rel = rng.integers(0, K, size=len(idx))
        used = rng.random(N) < 0.8
        t = lambda a: torch.from_numpy(a).to(DEV)
        x = torch.randn(N, Fin, device=DEV).to(feat_dtype)
        hmap = torch.where(torch.rand(R, device=DEV) < 0.4, torch.arange(R, device=DEV), torch.full((R,), -1, device=DEV))
        hbuf = torch.randn(R, H, device=DEV)
        g = torch.randn(R, H, device=DEV)
        res = {}
        for fused in (True, False):
            conv = MyRGCNConvHistory2(Fin, H, K, need_grad=True).to(DEV).train()
            with torch.no_grad():
                conv.linear.copy_(torch.randn(K, Fin, H, generator=torch.Generator().manual_seed(9)) * 0.1)
            conv.fused = fused
            xi = x.clone().requires_grad_(x_grad and feat_dtype == torch.float32)
            out, his = conv(xi, t(ptr), t(idx), t(rel), None, hmap if use_hist else None, hbuf if use_hist else None,
                            t(used), H if use_hist else 0, R)
            out.backward(g)
            res[fused] = (out.detach(), conv.linear.grad.clone(), None if xi.grad is None else xi.grad.clone(),
                          his.grad.clone() if (his.retains_grad or getattr(his, "_hc_grad_sink", False)) else None)
            want_count = np.bincount(rel, minlength=K + 1)
            want_count[0] = 0                                   # count_num skips value 0
            np.testing.assert_array_equal(conv.last_count.cpu().numpy(), want_count)
        tol = 2e-3 if feat_dtype == torch.float16 else 2e-5
        for a, b, what in zip(res[True], res[False], ("out", "weight grad", "input grad", "kept grad")):
            assert (a is None) == (b is None), what
            if a is not None:
                scale = float(b.abs().max()) or 1.0
                assert float((a - b).abs().max()) <= tol * scale, (what, R, Fin)
        if use_hist:
            hit = (hmap != -1).cpu().numpy()
            np.testing.assert_array_equal(res[True][0].cpu().numpy()[hit], hbuf.cpu().numpy()[hit])


def test_typed_csr_groups_edges_by_row_and_relation():
    from hiscache import typed_csr
    from helpers import random_csr
    rng = np.random.default_rng(9)
    R, N, K = 50, 40, 4
    ptr, idx = random_csr(rng, R + 10, N, 7)           # deeper-layer rows beyond the first R
    rel = rng.integers(0, K, size=len(idx))
    used = rng.random(N) < 0.8
    t = lambda a: torch.from_numpy(a).to(DEV)
    ptr2, idx2, cnt, deg = typed_csr(t(ptr), t(idx), t(rel), K, R, t(used))
    ptr2, idx2, cnt = ptr2.cpu().numpy(), idx2.cpu().numpy(), cnt.cpu().numpy()
    np.testing.assert_array_equal(deg.cpu().numpy(), np.diff(ptr)[:R])
    for r in range(R):
        for k in range(K):
            e = [j for j in range(ptr[r], ptr[r + 1]) if rel[j] == k and used[idx[j]]]
            v = r * K + k
            np.testing.assert_array_equal(idx2[ptr2[v]:ptr2[v + 1]], idx[e])
            assert cnt[r, k] == len(e)


@pytest.mark.parametrize("K,with_mask,short_types", [(5, True, False), (1, False, False), (64, True, True),
                                                      (7, False, True)])
def test_typed_csr_matches_oracle(orc, K, with_mask, short_types):
    """hc_typed_csr against the CPU checker: rows longer than one wave, relations and sources outside
    their ranges, relation arrays shorter than the edge list, with and without a used mask."""
    from helpers import random_csr
    rng = np.random.default_rng(50 + K)
    R, N = 700, 400
    ptr, idx = random_csr(rng, R + 50, N, 200, hub=5)
    idx = idx.copy()
    idx[rng.random(len(idx)) < 0.02] = N + 5
    rel = rng.integers(-1, K + 1, size=len(idx))
    if short_types:
        rel = rel[: int(ptr[R - 20])]
    used = (rng.random(N) < 0.7) if with_mask else None
    import hiscache_backend as be
    t = lambda a: None if a is None else torch.from_numpy(a).to(DEV)
    ptr2, idx2, cnt, deg, wts = be.typed_csr(t(ptr), t(idx), t(rel), K, R, N, t(used), want_weights=True)
    w_ptr2, w_idx2, w_cnt, w_deg = orc.typed_csr(ptr, idx, rel, K, R, N, used)
    np.testing.assert_array_equal(ptr2.cpu().numpy(), w_ptr2)
    np.testing.assert_array_equal(idx2.cpu().numpy()[: w_ptr2[-1]], w_idx2)
    np.testing.assert_array_equal(cnt.cpu().numpy(), w_cnt)
    np.testing.assert_array_equal(deg.cpu().numpy(), w_deg)
    # edge weights: 1/deg of the edge's row, so that the weighted sum over a group is its share of the mean
    np.testing.assert_array_equal(wts.cpu().numpy()[: w_ptr2[-1]], orc.typed_csr_weights(w_ptr2, w_deg, K))
    again = be.typed_csr(t(ptr), t(idx), t(rel), K, R, N, t(used))
    assert len(again) == 4 and torch.equal(again[1][: w_ptr2[-1]], idx2[: w_ptr2[-1]])
    p0 = be.typed_csr(t(ptr), t(idx), t(rel), K, 0, N, t(used))[0]
    assert p0.cpu().tolist() == [0]
    with pytest.raises(ValueError):
        be.typed_csr(t(ptr), t(idx), t(rel), 65, R, N, t(used))


def test_typed_csr_library_scan_path_agrees(orc):
    """Above 2^20 (row, relation) groups the group offsets come from the library's scan instead of the count
    kernel's last block: same result as the CPU checker, and as the small path on a prefix of the rows."""
    from helpers import random_csr
    import hiscache_backend as be
    rng = np.random.default_rng(77)
    R, N, K = 17_000, 5000, 64
    assert R * K > be.TYPED_CSR_SMALL_GROUPS
    ptr, idx = random_csr(rng, R, N, 6)
    rel = rng.integers(0, K, size=len(idx))
    t = lambda a: torch.from_numpy(a).to(DEV)
    got = be.typed_csr(t(ptr), t(idx), t(rel), K, R, N, None, want_weights=True)
    w_ptr2, w_idx2, w_cnt, w_deg = orc.typed_csr(ptr, idx, rel, K, R, N, None)
    np.testing.assert_array_equal(got[0].cpu().numpy(), w_ptr2)
    np.testing.assert_array_equal(got[1].cpu().numpy()[: w_ptr2[-1]], w_idx2)
    np.testing.assert_array_equal(got[2].cpu().numpy(), w_cnt)
    np.testing.assert_array_equal(got[4].cpu().numpy()[: w_ptr2[-1]], orc.typed_csr_weights(w_ptr2, w_deg, K))
    R2 = 12_000                                                   # 768 000 groups: scanned by the count kernel
    small = be.typed_csr(t(ptr), t(idx), t(rel), K, R2, N, None)
    assert torch.equal(small[0], got[0][: R2 * K + 1]) and torch.equal(small[2], got[2][:R2])
    n_small = int(small[0][-1])
    assert torch.equal(small[1][:n_small], got[1][:n_small])
    torch.cuda.synchronize()
    assert int(be._ticket(torch.device(DEV)).abs().sum()) == 0


def test_count_num_few_and_many_bins(orc):
    import hiscache_backend as be
    rng = np.random.default_rng(61)
    for n, mmax in ((0, 3), (5, 1), (300_000, 5), (300_000, 4095), (100_000, 6000)):
        arr = rng.integers(0, mmax + 1, size=n)
        got = be.count_num(torch.from_numpy(arr).to(DEV), mmax).cpu().numpy()
        np.testing.assert_array_equal(got, orc.count_num(arr, mmax))


def test_edge_types_by_ranges_matches_oracle(orc):
    import hiscache_backend as be
    from helpers import random_csr
    rng = np.random.default_rng(72)
    R, n_all = 900, 1500
    ptr, idx = random_csr(rng, R + 100, n_all, 150, hub=4)
    idx = idx.copy()
    idx[rng.random(len(idx)) < 0.01] = n_all + 3
    s2f = rng.permutation(100_000)[:n_all]
    bounds = np.array([30_000, 65_000])
    table = np.array([[0, 1, -1], [2, -1, 3], [-1, 4, -1]])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int64)).to(DEV)
    got = be.edge_types_by_ranges(t(ptr), t(idx), t(s2f), R, t(bounds), t(table)).cpu().numpy()
    np.testing.assert_array_equal(got, orc.edge_types_by_ranges(ptr, idx, s2f, R, bounds, table))
    none = be.edge_types_by_ranges(t(ptr), t(idx), t(s2f), R, t(np.zeros(0)), t(np.array([[7]]))).cpu().numpy()
    assert set(np.unique(none[: ptr[R]])) <= {7, -1}


def test_evict_matches_oracle(orc):
    """hc_evict (gradient rule + staleness rule in one launch) against the CPU statement of
    HistoryTable.evict_by_both, and the staleness rule alone."""
    import hiscache_backend as be
    from oracle import host_model
    rng = np.random.default_rng(81)
    cap, N, M = 5000, 20000, 3000
    for trial in range(4):
        owners = rng.choice(N, size=4000, replace=False)
        slots = rng.choice(cap, size=4000, replace=False)
        h2f = np.full(cap, -1, np.int64); f2h = np.full(N, -1, np.int64); chk = np.full(cap, -1, np.int64)
        h2f[slots] = owners; f2h[owners] = slots; chk[slots] = rng.integers(0, 30, size=4000)
        nodes = rng.choice(N, size=M, replace=False)
        s2h = f2h[nodes].copy()
        s2h[:100] = -1
        score = rng.random(M).astype(np.float32)
        score[5:9] = score[4]                                      # ties around the threshold side
        dev = [torch.from_numpy(a.copy()).to(DEV) for a in (chk, h2f, f2h)]
        cpu = [torch.from_numpy(a.copy()) for a in (chk, h2f, f2h)]
        if trial % 2 == 0:
            thres = host_model.evict_by_both(cpu[0], cpu[1], cpu[2], torch.from_numpy(s2h), torch.from_numpy(score),
                                             rate=0.25, glb_iter=30, staleness_thres=12)
            be.evict(dev[0], dev[1], dev[2], 30 - 12, sub2slot=torch.from_numpy(s2h).to(DEV),
                     score=torch.from_numpy(score).to(DEV),
                     thres=torch.tensor([float(thres)], dtype=torch.float32, device=DEV))
        else:
            host_model.evict_by_staleness(cpu[0], cpu[1], cpu[2], 30, 12)
            be.evict(dev[0], dev[1], dev[2], 30 - 12)
        for d, c in zip(dev, cpu):
            np.testing.assert_array_equal(d.cpu().numpy(), c.numpy())
        assert (cpu[1] != -1).sum() < 4000
