"""Seeded sweeps over many small random configurations of every entry point, against the CPU checker.

Each sweep draws its cases from one master seed, so the set of cases is fixed; a failure names the
case seed, which rebuilds the inputs.  Widths on and off the fast paths, fp32/fp16/bf16 inputs and
tables, empty rows, rows above the long-row threshold, hub sources, history fractions 0 / 0.3 / 1,
single- and multi-head weights, ring wrap-around with capacity 1 upwards, relation counts up to 64,
cache buffers from two rows upwards, graphs with multi-edges and isolated nodes.  Bars as elsewhere:
bit-exact except the edge gradient (dot products in another order: 1e-5 of the sum of magnitudes)
and the reduced-precision input gradients (1e-2)."""
import os

import numpy as np
import pytest
import torch

from helpers import layered_batch, random_csr, random_hmap
from test_oracle_sampler import check_batch, simple_graph

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
WIDTHS = [1, 2, 3, 4, 7, 8, 16, 17, 32, 60, 64, 65, 96, 100, 128, 160, 172, 192, 200, 256, 300, 320, 384, 448,
          512, 576, 640, 704, 768, 832, 1000, 1024, 1088, 1536, 2048]
TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
eq = np.testing.assert_array_equal


def T(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    return t.to(dtype) if dtype is not None else t


def none():
    return torch.empty(0, device=DEV)


@pytest.fixture(scope="module")
def be():
    import hiscache_backend
    hiscache_backend.load_library()
    return hiscache_backend


def case_seeds(master_seed, n):
    # HISCACHE_SWEEP_SHIFT=k draws another fixed set of cases (for a longer sweep on demand)
    shift = int(os.environ.get("HISCACHE_SWEEP_SHIFT", "0"))
    return [int(s) for s in np.random.default_rng(master_seed + 1000 * shift).integers(1 << 30, size=n)]


# ------------------------------------------------------------------------------ aggregation
def aggregation_case(be, orc, s):
    rng = np.random.default_rng(s)
    F = int(rng.choice(WIDTHS))
    dt = [torch.float32, torch.float32, torch.float16, torch.bfloat16][int(rng.integers(4))]
    R = int(rng.choice([1, 2, 63, 64, 65, 300, 1000, 5000, 20000]))
    N = int(rng.choice([1, 5, 100, 777, 4000]))
    R = max(1, min(R, int(4e6 // F)))
    maxdeg = int(rng.choice([1, 3, 12, 40]))
    hub = [None, 70, 300, 1500][int(rng.integers(4))]
    kind = int(rng.integers(3))
    frac = float(rng.choice([0.0, 0.3, 1.0]))
    ptr, idx = random_csr(rng, R, N, maxdeg, hub=hub)
    E = len(idx)
    x = T(rng.standard_normal((N, F)).astype(np.float32), dt)
    x32 = x.float().cpu().numpy()
    g = rng.standard_normal((R, F)).astype(np.float32)
    split = be.long_row_edges(F, dt)
    if kind == 0:        # mean with per-row substitution, history rows at least as wide as the features
        hs = F if rng.random() < 0.7 else F + int(rng.integers(1, 9)) * 8
        hmap = random_hmap(rng, R, frac)
        hb = T(rng.standard_normal((R, hs)).astype(np.float32), dt)
        xt, hbt = x.clone().requires_grad_(True), hb.clone().requires_grad_(True)
        out = be.aggr_forward_history(xt, T(ptr), T(idx), T(hmap), hbt, hs, R)
        eq(out.detach().cpu().numpy(), orc.fwd_mean_row(ptr, idx, x32, hmap, hb.float().cpu().numpy(), split_above=split))
        out.backward(T(g))
        gx, gh = orc.bwd_mean_row(ptr, idx, g, hmap, N, hbuf_shape=(R, hs), chunk=be.bwd_chunk_edges(F))
        gxg, ghg = xt.grad.float().cpu().numpy(), hbt.grad.float().cpu().numpy()
        if dt == torch.float32:
            eq(gxg, gx)
            eq(ghg, gh)
        else:
            np.testing.assert_allclose(gxg, gx, rtol=1e-2, atol=1e-2 * max(1.0, float(np.abs(gx).max())))
            np.testing.assert_allclose(ghg, gh, rtol=1e-2, atol=1e-2)
    elif kind == 1:      # mean with per-source substitution
        hist = T(rng.standard_normal((64, F)).astype(np.float32), dt)
        smap = np.where(rng.random(N) < frac, rng.integers(0, 64, size=N), -1).astype(np.int64)
        out = be.aggr_forward_source_history(x, T(ptr), T(idx), T(smap), hist)
        eq(out.cpu().numpy(), orc.fwd_mean_src(ptr, idx, x32, smap, hist.float().cpu().numpy(), split_above=split))
    elif E > 0:          # weighted sums, one or several heads
        H = int(rng.choice([1, 1, 2, 3]))
        if H * F * max(N, R) > 6e6:
            H = 1
        multi = H > 1
        vin = rng.standard_normal((N, H, F) if multi else (N, F)).astype(np.float32)
        ev = rng.standard_normal((E, H) if multi else (E,)).astype(np.float32)
        gg = rng.standard_normal((R, H, F) if multi else (R, F)).astype(np.float32)
        hkind = int(rng.integers(3))
        if hkind == 0:
            hmap, hbuf, hsz = None, None, 0
        else:
            hsz = F * H if (hkind == 2 and multi) else F
            hmap = random_hmap(rng, R, frac)
            hbuf = rng.standard_normal((R, hsz)).astype(np.float32)
        xt, evt = T(vin).requires_grad_(True), T(ev).requires_grad_(True)
        hbt = None if hbuf is None else T(hbuf).requires_grad_(True)
        out = be.aggr_forward_history_edge_value(xt, T(ptr), T(idx), evt, none() if hmap is None else T(hmap),
                                                 none() if hbt is None else hbt, hsz, R)
        eq(out.detach().cpu().numpy(),
           orc.fwd_edge_value(ptr, idx, ev, vin, hmap, hbuf, split_above=0 if multi else be.long_row_edges(F)))
        out.backward(T(gg))
        gx, gh, eg = orc.bwd_edge_value(ptr, idx, ev, gg, hmap, vin, N, hsize=hsz, want_edge_grad=True)
        eq(xt.grad.cpu().numpy(), gx)
        if hbt is not None:
            eq(hbt.grad.cpu().numpy(), gh)
        dst = np.repeat(np.arange(R), np.diff(ptr))
        scale = (np.abs(gg[dst]) * np.abs(vin[idx])).sum(-1)
        assert (np.abs(evt.grad.cpu().numpy() - eg) <= 1e-5 * scale + 1e-7).all()


def test_sweep_aggregation(be, orc):
    for i, s in enumerate(case_seeds(101, 400)):
        try:
            aggregation_case(be, orc, s)
        except AssertionError as e:
            raise AssertionError("aggregation case %d (seed %d): %s" % (i, s, str(e)[:600])) from None


# ------------------------------------------------------------------------------ admission, grouping, views
def admission_case(be, orc, rng):
    F = int(rng.choice([1, 3, 4, 17, 64, 100, 128, 172, 192, 255, 256, 300, 512, 768, 1000, 1024, 1500, 2048]))
    dtype = ["f32", "f16", "bf16"][int(rng.integers(3))]
    N = int(rng.choice([50, 3000, 40000]))
    cap = min(int(rng.choice([1, 7, 100, 700, 5000])), N)
    M = min(int(rng.choice([1, 31, 32, 33, 64, 1000, 4097])), N)
    M = max(1, min(M, int(3e6 // F)))
    nk = [orc.NORM_L2, orc.NORM_L1][int(rng.integers(2))]
    use_used, use_age = rng.random() < 0.7, rng.random() < 0.7
    code = {"f32": orc.DT_F32, "f16": orc.DT_F16, "bf16": orc.DT_BF16}[dtype]
    ref = dict(table=np.zeros((cap, F), np.float32 if dtype == "f32" else np.uint16), f2s=np.full(N, -1, np.int64),
               s2f=np.full(cap, -1, np.int64), checkin=np.full(cap, -1, np.int64), header=np.zeros(1, np.int64))
    ref["header"][0] = int(rng.integers(0, cap))
    dev = {k: T(v) for k, v in ref.items()}
    if dtype != "f32":
        dev["table"] = dev["table"].view(TORCH_DT[dtype])
    for it in range(4):
        ck = [orc.CMP_LT, orc.CMP_NOT_GT][int(rng.integers(2))]
        nodes = rng.choice(N, size=M, replace=False).astype(np.int64)
        grad = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
        emb = rng.standard_normal((M, F)).astype(np.float32)
        slot = ref["f2s"][nodes].copy()
        age = rng.integers(0, 21, size=M).astype(np.int32) if use_age else None
        used = (rng.random(M) < 0.9) if use_used else None
        thres = float(np.sort(orc.row_scores(grad, nk))[int(rng.integers(0, M))])   # one score equals the threshold
        rmask, rscore, rslots = orc.grad_check(grad, emb, slot, age, used, nodes, thres, 10, nk, ck, ref["table"], code,
                                               ref["f2s"], ref["s2f"], ref["checkin"], ref["header"], it)
        mask, score, slots = be.grad_check(T(grad), T(emb), T(slot), T(nodes), torch.tensor([thres], device=DEV),
                                           dev["table"], dev["f2s"], dev["s2f"], dev["header"], it,
                                           age=None if age is None else T(age), age_limit=10,
                                           used=None if used is None else T(used), checkin=dev["checkin"],
                                           norm_kind=nk, cmp_kind=ck, want_slots=True)
        eq(mask.cpu().numpy(), rmask)
        eq(score.cpu().numpy(), rscore)
        if int(rmask.sum()) <= cap:
            eq(slots.cpu().numpy(), rslots)
        for k in ("f2s", "s2f", "checkin", "header"):
            eq(dev[k].cpu().numpy(), ref[k], err_msg=k)
        tab = dev["table"] if dtype == "f32" else dev["table"].view(torch.int16)
        live = ref["s2f"] != -1
        eq(tab.cpu().numpy().view(ref["table"].dtype)[live], ref["table"][live])


def typed_csr_case(be, orc, rng):
    R = int(rng.choice([1, 64, 300, 5000, 60000]))
    N = int(rng.choice([1, 100, 4000, 100000]))
    K = int(rng.choice([1, 2, 5, 8, 33, 64]))
    ptr, idx = random_csr(rng, R, N, int(rng.choice([1, 3, 12, 40])), hub=[None, 300, 1500][int(rng.integers(3))])
    rel = rng.integers(0, K, size=len(idx)).astype(np.int64)
    used = (rng.random(N) < 0.7) if rng.random() < 0.5 else None
    got = [a.cpu().numpy() for a in be.typed_csr(T(ptr), T(idx), T(rel), K, R, N, used_mask=None if used is None else T(used))]
    want = orc.typed_csr(ptr, idx, rel, K, R, N, used_mask=used)
    eq(got[0], want[0])
    eq(got[1][: len(want[1])], want[1])
    eq(got[2].reshape(-1), want[2].reshape(-1))
    eq(got[3], want[3])


def transposed_view_case(be, orc, rng):
    R = int(rng.choice([1, 64, 300, 5000, 200000]))
    N = int(rng.choice([1, 100, 4000, 1000000]))
    ptr, idx = random_csr(rng, R, N, int(rng.choice([1, 3, 12])), hub=[None, 300, 5000][int(rng.integers(3))])
    hmap = random_hmap(rng, R, float(rng.choice([0.0, 0.3, 1.0]))) if rng.random() < 0.6 else None
    ptrT, rowT, edgeT = be.build_transpose(T(ptr), T(idx), None if hmap is None else T(hmap), R, N)
    wp, wr, we = orc.build_transpose(ptr, idx, hmap, N)
    eq(ptrT.cpu().numpy(), wp)
    eq(rowT.cpu().numpy()[: len(wr)], wr)
    eq(edgeT.cpu().numpy()[: len(we)], we)


def used_masks_case(be, orc, rng):
    L = int(rng.integers(1, 4))
    n_seed = int(rng.choice([1, 7, 100, 1000]))
    b = layered_batch(rng, 20000, n_seed, [int(rng.choice([2, 5, 10])) for _ in range(L)])
    ptr, idx, nnl = b["ptr"], b["idx"], b["num_node_in_layer"]
    n_all, n1 = int(nnl[-1]), int(nnl[1])
    hmap = np.full(n1, -1, np.int64)
    hmap[rng.random(n1) < float(rng.choice([0.0, 0.35, 1.0]))] = 5
    got = be.count_history_reconstruct(T(ptr), T(idx), T(hmap), n_all, n_seed, L)
    for a, r in zip(got, orc.count_history_reconstruct(ptr, idx, hmap, n_all, n_seed, L)):
        eq(a.cpu().numpy(), r)


def test_sweep_admission_grouping_views(be, orc):
    kinds = [admission_case, typed_csr_case, transposed_view_case, used_masks_case]
    for i, s in enumerate(case_seeds(102, 1200)):
        rng = np.random.default_rng(s)
        case = kinds[int(rng.integers(4))]
        try:
            case(be, orc, rng)
        except AssertionError as e:
            raise AssertionError("%s %d (seed %d): %s" % (case.__name__, i, s, str(e)[:600])) from None


# ------------------------------------------------------------------------------ cache policy, sampler
def cache_case(orc, rng):
    from hiscache import HistoryCache, PinnedFeatureStore, make_config
    from hiscache.synthetic import make_batch
    from oracle import host_model
    N = int(rng.choice([500, 3000, 20000]))
    Fin, H = int(rng.choice([16, 32, 100, 128])), int(rng.choice([32, 48, 64, 256]))
    rows, n_seed, L = int(rng.choice([2, 50, 400, 3000])), int(rng.choice([1, 10, 40, 200])), 3
    fan = [int(rng.choice([2, 4, 6, 10])) for _ in range(L)]
    rate, stale = float(rng.choice([0.3, 0.6, 0.95])), int(rng.choice([2, 4, 100]))
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    hot = rng.permutation(N).astype(np.int64)
    buffer_floats = int(rows * np.lcm(Fin, H))
    cfg = make_config(Fin, 7, H, L, method="grad", rate=rate, staleness_thres=stale, device=DEV)
    cache = HistoryCache(PinnedFeatureStore(feats, device=DEV), cfg, "history_uvm", total_num_node=N,
                         buffer_bytes=buffer_floats * 4, hot_ids=hot)
    st = host_model.new_cache_state(N, Fin, H, buffer_floats, hot, feats)
    for it in range(1, 5):
        b = layered_batch(rng, N, n_seed, fan)
        labels = rng.integers(0, 7, size=N)
        gpu, cpu = make_batch(b, labels, DEV), make_batch(b, labels, "cpu")
        cache.lookup_and_load(gpu, L)
        ref = host_model.lookup_and_load(st, cpu, L, feats)
        eq(cache.sub2embed.cpu().numpy(), ref.sub2embed.numpy())
        eq(cache.sub2feat.cpu().numpy(), ref.sub2feat.numpy())
        for a, r in zip(cache.used_masks, ref.used_masks):
            eq(a.cpu().numpy(), r.numpy())
        eq(cache.load_mask.cpu().numpy(), ref.load_mask.numpy())
        eq(gpu.x.cpu().numpy(), ref.x.numpy())
        eq(cache.cached_embedding.cpu().numpy(), ref.cached_embedding.numpy())
        n1 = int(cpu.num_node_in_layer[1])
        emb = rng.standard_normal((n1, H)).astype(np.float32)
        grad = (rng.standard_normal((n1, H)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)
        pe = torch.from_numpy(emb).to(DEV).requires_grad_(True)
        pe.grad = torch.from_numpy(grad).to(DEV)
        cache.produced_embedding = pe
        cache.update_history(gpu, it)
        mask, _ = host_model.update_history(st, cpu.sub_to_full, ref.sub2embed, torch.from_numpy(emb),
                                            torch.from_numpy(orc.row_scores(grad)), rate, stale, it)
        eq(cache.last_record_mask.cpu().numpy(), mask.numpy())
        eq(cache.full2embed.cpu().numpy(), st.full2embed.numpy())
        eq(cache.embed2full.cpu().numpy(), st.embed2full.numpy())
        eq(cache.feat2full.cpu().numpy(), st.feat2full.numpy())
        assert cache.header == st.header
        eq(cache.buffer.view(-1, H)[: st.header].cpu().numpy(), st.buffer.view(-1, H)[: st.header].numpy())


def sampler_case(orc, rng):
    from hiscache import NeighborSampler
    n = int(rng.choice([50, 2000, 12000]))
    max_deg, hubs = int(rng.choice([1, 5, 30])), int(rng.choice([0, 3]))
    fan = [int(rng.choice([1, 2, 5, 15, 40])) for _ in range(int(rng.integers(1, 5)))]
    n_seed = min(int(rng.choice([1, 13, 200, 1000])), n)
    simple = rng.random() >= 0.3
    if simple:
        indptr, indices = simple_graph(rng, n, min(max_deg, n - 1), hubs=hubs if n > 100 else 0)
    else:                # repeated neighbours and nodes without neighbours
        deg = rng.integers(0, max_deg + 1, size=n)
        deg[: n // 10] = 0
        indptr = np.zeros(n + 1, np.int64)
        np.cumsum(deg, out=indptr[1:])
        indices = rng.integers(0, max(1, n // 4), size=int(indptr[-1])).astype(np.int64)
    sampler = NeighborSampler(indptr, indices, fan, seed=int(rng.integers(1 << 20)), device=DEV)
    for it in range(3):  # consecutive batches share the node map
        seeds = rng.choice(n, size=n_seed, replace=False).astype(np.int64)
        batch = sampler.sample(torch.from_numpy(seeds).to(DEV))
        want = orc.sample_layers(indptr, indices, seeds, fan, sampler.batch_seed(it))
        got = {"ptr": batch.ptr.cpu().numpy(), "idx": batch.idx.cpu().numpy(),
               "sub_to_full": batch.sub_to_full.cpu().numpy(), "num_node_in_layer": batch.num_node_in_layer.numpy(),
               "num_edge_in_layer": np.asarray(batch.num_edge_in_layer)}
        for k in want:
            eq(got[k], want[k], err_msg=k)
        if simple:
            check_batch(got, indptr, indices, seeds, fan)
    assert int((sampler.node_map != 0x7fffffff).sum()) == 0


def test_sweep_cache_policy_and_sampler(orc):
    for i, s in enumerate(case_seeds(103, 240)):
        rng = np.random.default_rng(s)
        case = [cache_case, sampler_case][int(rng.integers(2))]
        try:
            case(orc, rng)
        except AssertionError as e:
            raise AssertionError("%s %d (seed %d): %s" % (case.__name__, i, s, str(e)[:600])) from None


# ------------------------------------------------------------------------------ row gathers
def row_gather_case(be, s):
    """Masked row gathers of a matrix in device memory, in pinned host memory and in two tiers, and the fix-up of a
    guessed gather, against NumPy indexing: the values are copies (or conversions of one element), so every bit
    must agree."""
    rng = np.random.default_rng(s)
    F = int(rng.choice(WIDTHS[:31]))
    src_dt, out_dt = [("f32", "f32"), ("f32", "f32"), ("f16", "f16"), ("f16", "f32"), ("bf16", "f32"),
                      ("f32", "f16")][int(rng.integers(6))]
    N = int(rng.choice([1, 2, 50, 777, 4000]))
    n = int(rng.choice([1, 15, 16, 17, 63, 64, 65, 255, 256, 257, 1000, 3000]))
    n = max(1, min(n, int(3e6 // F)))
    src = torch.from_numpy(rng.standard_normal((N, F)).astype(np.float32)).to(TORCH_DT[src_dt])
    host = torch.empty(src.shape, dtype=src.dtype, pin_memory=True)
    host.copy_(src)
    dev = src.to(DEV)
    ids_np = rng.integers(-N, N, size=n)                             # negative ids address from the end
    if n > 4:
        ids_np[int(rng.integers(n))] = N + int(rng.integers(3))      # outside the matrix: a cleared row
        ids_np[int(rng.integers(n))] = -N - 1 - int(rng.integers(3))
    masked = rng.random() < 0.7
    mask_np = rng.random(n) < rng.choice([0.0, 0.3, 0.9, 1.0]) if masked else np.ones(n, bool)
    ids, mask = T(ids_np), (T(mask_np) if masked else None)
    wrapped = np.where(ids_np < 0, ids_np + N, ids_np)
    inside = (wrapped >= 0) & (wrapped < N)
    take = inside & mask_np
    want = src[torch.from_numpy(np.where(inside, wrapped, 0))].to(TORCH_DT[out_dt])
    want[torch.from_numpy(~take)] = 0
    for matrix in (dev, host):
        got = be.gather_rows(matrix, ids, mask=mask, out_dtype=TORCH_DT[out_dt])
        assert torch.equal(got.cpu(), want), ("gather", matrix.is_cuda)
    # two tiers
    k = int(N * rng.choice([0.0, 0.4, 1.0]))
    hot_ids = T(rng.permutation(N)[:k].copy())
    slot = torch.full((N,), -1, dtype=torch.int32, device=DEV)
    slot[hot_ids] = torch.arange(k, dtype=torch.int32, device=DEV)
    hot = dev[hot_ids].contiguous() if k else torch.empty((0, F), dtype=dev.dtype, device=DEV)
    out = torch.full((n, F), 5.0, dtype=TORCH_DT[out_dt], device=DEV)
    _, cold = be.gather_rows_hot(hot, slot, ids, mask=mask, out=out)
    slot_np = slot.cpu().numpy()
    eq(cold.cpu().numpy().astype(bool), take & (slot_np[np.where(inside, wrapped, 0)] < 0))
    be.gather_rows_flagged(host, ids, cold, out)
    assert torch.equal(out.cpu(), want), "tiers"
    # a gather under a guess, brought to the exact mask
    guess_np = rng.random(n) < 0.5
    rows = be.gather_rows(host, ids, mask=T(guess_np), out_dtype=TORCH_DT[out_dt])
    be.fixup_rows(host, ids, T(mask_np), T(guess_np), rows)
    assert torch.equal(rows.cpu(), want), "fixup"


def test_sweep_row_gathers(be):
    for s in case_seeds(44, 400):
        try:
            row_gather_case(be, s)
        except Exception as e:                     # name the case: its seed rebuilds the inputs
            raise AssertionError(f"row gather case seed {s}: {e}") from e
