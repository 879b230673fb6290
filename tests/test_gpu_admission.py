"""GPU parity of the used-mask, score and admission kernels against the CPU oracle (bit-exact:
masks, slot ids, maps, header; table rows exact because fp32->fp16/bf16 rounding is deterministic)."""
import numpy as np
import pytest
import torch

from helpers import layered_batch, random_csr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    return t.to(dtype) if dtype is not None else t


@pytest.fixture(scope="module")
def be():
    import hiscache_backend
    hiscache_backend.load_library()
    return hiscache_backend


@pytest.mark.parametrize("seed,L,fanout,n_seed", [(0, 2, [10, 5], 100), (1, 3, [15, 10, 5], 60), (2, 1, [6], 20),
                                                   (3, 3, [2, 2, 2], 7)])
def test_count_history_bit_exact(be, orc, seed, L, fanout, n_seed):
    rng = np.random.default_rng(seed)
    b = layered_batch(rng, 5000, n_seed, fanout)
    ptr, idx, nnl = b["ptr"], b["idx"], b["num_node_in_layer"]
    n_all, n1 = int(nnl[-1]), int(nnl[1])
    hmap = np.full(n1, -1, np.int64)
    hmap[rng.random(n1) < 0.35] = 5
    for hm in (hmap, None):
        got = be.count_history_reconstruct(T(ptr), T(idx), torch.empty(0, device=DEV) if hm is None else T(hm),
                                           n_all, n_seed, L)
        ref = orc.count_history_reconstruct(ptr, idx, hm, n_all, n_seed, L)
        assert len(got) == L + 1
        for a, r in zip(got, ref):
            assert a.dtype == torch.bool
            np.testing.assert_array_equal(a.cpu().numpy(), r)


@pytest.mark.parametrize("F", [1, 3, 64, 128, 255, 256, 300, 512, 768, 1024, 1500])
@pytest.mark.parametrize("kind", ["l2", "l1"])
def test_row_scores_bit_exact(be, orc, F, kind):
    rng = np.random.default_rng(F)
    M = 203
    g = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
    k = be.NORM_L2 if kind == "l2" else be.NORM_L1
    got = be.row_scores(T(g), k).cpu().numpy()
    np.testing.assert_array_equal(got, orc.row_scores(g, k))


def fresh_ring(N, cap, F, dtype):
    return dict(table=np.zeros((cap, F), np.float32 if dtype == "f32" else np.uint16),
                f2s=np.full(N, -1, np.int64), s2f=np.full(cap, -1, np.int64),
                checkin=np.full(cap, -1, np.int64), header=np.zeros(1, np.int64))


TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("F", [256, 100])
def test_grad_check_fused_bit_exact(be, orc, dtype, F):
    rng = np.random.default_rng(11)
    N, cap, M = 5000, 700, 1000
    code = {"f32": orc.DT_F32, "f16": orc.DT_F16, "bf16": orc.DT_BF16}[dtype]
    ref = fresh_ring(N, cap, F, dtype)
    ref["header"][0] = cap - 50
    dev = {k: T(v) for k, v in ref.items()}
    if dtype != "f32":
        dev["table"] = dev["table"].view(TORCH_DT[dtype])
    for it, cmp_kind in enumerate([orc.CMP_LT, orc.CMP_NOT_GT, orc.CMP_LT, orc.CMP_LT]):
        sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int64)
        grad = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
        emb = rng.standard_normal((M, F)).astype(np.float32)
        slot = ref["f2s"][sub_to_full].copy()
        age = rng.integers(0, 21, size=M).astype(np.int32)
        used = rng.random(M) < 0.9
        thres = float(np.sort(orc.row_scores(grad))[M // 2])       # one score equals the threshold
        rmask, rscore, rslots = orc.grad_check(grad, emb, slot, age, used, sub_to_full, thres, 10,
                                               orc.NORM_L2, cmp_kind, ref["table"], code, ref["f2s"],
                                               ref["s2f"], ref["checkin"], ref["header"], it)
        mask, score, slots = be.grad_check(T(grad), T(emb), T(slot), T(sub_to_full),
                                           torch.tensor([thres], device=DEV), dev["table"], dev["f2s"],
                                           dev["s2f"], dev["header"], it, age=T(age), age_limit=10,
                                           used=T(used), checkin=dev["checkin"], cmp_kind=cmp_kind,
                                           want_slots=True)
        np.testing.assert_array_equal(mask.cpu().numpy(), rmask)
        np.testing.assert_array_equal(score.cpu().numpy(), rscore)
        np.testing.assert_array_equal(slots.cpu().numpy(), rslots)
        for k in ("f2s", "s2f", "checkin", "header"):
            np.testing.assert_array_equal(dev[k].cpu().numpy(), ref[k], err_msg=k)
        tab = dev["table"] if dtype == "f32" else dev["table"].view(torch.int16)
        live = ref["s2f"] != -1
        np.testing.assert_array_equal(tab.cpu().numpy().view(ref["table"].dtype)[live], ref["table"][live])


def test_grad_check_more_admitted_than_capacity(be, orc):
    rng = np.random.default_rng(12)
    N, F, cap, M = 3000, 64, 100, 1000
    ref = fresh_ring(N, cap, F, "f32")
    ref["header"][0] = 33
    # some nodes are cached already and stale, so they are re-admitted
    pre = rng.choice(N, size=cap, replace=False)
    ref["f2s"][pre] = np.arange(cap)
    ref["s2f"][:] = pre
    dev = {k: T(v) for k, v in ref.items()}
    sub_to_full = np.concatenate([pre[:40], rng.choice(np.setdiff1d(np.arange(N), pre), M - 40, replace=False)])
    rng.shuffle(sub_to_full)
    slot = ref["f2s"][sub_to_full].copy()
    age = np.full(M, 50, np.int32)
    emb = rng.standard_normal((M, F)).astype(np.float32)
    score = rng.random(M).astype(np.float32)
    rmask, _, rslots = orc.grad_check(None, emb, slot, age, None, sub_to_full, 0.8, 10, orc.NORM_L2, orc.CMP_LT,
                                      ref["table"], orc.DT_F32, ref["f2s"], ref["s2f"], ref["checkin"],
                                      ref["header"], 9, score_in=score)
    assert rmask.sum() > 3 * cap
    mask, _, slots = be.grad_check(None, T(emb), T(slot), T(sub_to_full), torch.tensor([0.8], device=DEV),
                                   dev["table"], dev["f2s"], dev["s2f"], dev["header"], 9, age=T(age),
                                   age_limit=10, checkin=dev["checkin"], score=T(score), want_slots=True)
    np.testing.assert_array_equal(mask.cpu().numpy(), rmask)
    np.testing.assert_array_equal(slots.cpu().numpy(), rslots)
    for k in ("f2s", "s2f", "checkin", "header", "table"):
        np.testing.assert_array_equal(dev[k].cpu().numpy(), ref[k], err_msg=k)


def test_record_history_reference_signature(be, orc):
    rng = np.random.default_rng(13)
    N, cap, hs = 4000, 300, 128
    ref = dict(buf=np.zeros((cap, hs), np.float32), h2f=np.full(cap, -1, np.int64),
               f2h=np.full(N, -1, np.int64), checkin=np.full(cap, -1, np.int64), header=np.zeros(1, np.int64))
    dev = {k: T(v) for k, v in ref.items()}
    for it in range(5):
        M = int(rng.integers(100, 400))
        sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int64)
        new = rng.standard_normal((M, hs)).astype(np.float32)
        score = rng.random(M).astype(np.float32)
        thres = np.float32(0.0) if it == 3 else np.float32(np.sort(score)[int(0.7 * (M - 1))])
        used = rng.random(M) < 0.8
        sub2hist = ref["f2h"][sub_to_full].copy()
        sub2hist[: M // 5] = -1
        orc.record_history(new, ref["buf"], used, sub_to_full, sub2hist, ref["h2f"], ref["f2h"], ref["header"],
                           score, thres, ref["checkin"], it)
        be.record_history(T(new), dev["buf"], T(used), T(sub_to_full), T(sub2hist), dev["h2f"], dev["f2h"],
                          dev["header"], T(score), torch.tensor([thres], device=DEV), dev["checkin"], it)
        for k in ref:
            np.testing.assert_array_equal(dev[k].cpu().numpy(), ref[k], err_msg=f"{k} iter {it}")


@pytest.mark.parametrize("seed,n_seed,depth,kids", [(1, 5, 3, 4), (2, 400, 2, 7), (3, 1, 4, 3), (4, 300, 3, 6)])
def test_structure_score_on_forests(be, seed, n_seed, depth, kids):
    """On a forest of depth <= num_layer the reference's get_graph_structure_score
    (src/cpp/src/grad_check.cu:132-163) has one possible result, the product of the ancestors'
    degrees: the device kernel must give it."""
    from test_oracle_admission import random_forest_batch
    rng = np.random.default_rng(seed)
    ptr, idx, n_nodes, want = random_forest_batch(rng, n_seed, depth, kids)
    expect = np.zeros(n_nodes + 2, np.int64)
    for v, prod in want.items():
        expect[v] = prod
    got = be.get_graph_structure_score(T(ptr), T(idx), n_nodes + 2, n_seed, depth)
    np.testing.assert_array_equal(got.cpu().numpy(), expect)


def test_small_helpers(be, orc):
    rng = np.random.default_rng(14)
    arr = rng.integers(0, 6, size=100000)
    np.testing.assert_array_equal(be.count_num(T(arr), 5).cpu().numpy(), orc.count_num(arr, 5))
    b = layered_batch(rng, 3000, 30, [5, 4, 3])
    got = be.get_graph_structure_score(T(b["ptr"]), T(b["idx"]), int(b["num_node_in_layer"][-1]), 30, 3)
    ref = orc.get_graph_structure_score(b["ptr"], b["idx"], int(b["num_node_in_layer"][-1]), 30, 3)
    np.testing.assert_array_equal(got.cpu().numpy(), ref)
    table = rng.standard_normal((50, 96)).astype(np.float32)
    ids = rng.integers(-1, 50, size=200)
    mask = rng.random(200) < 0.7
    np.testing.assert_array_equal(be.gather_rows(T(table), T(ids), T(mask)).cpu().numpy(),
                                  orc.gather_rows(table, ids, mask))
    # zero-copy read of pinned host memory, fp16 source, accumulate
    host = torch.from_numpy(table).half().pin_memory()
    out = torch.ones((200, 96), device=DEV)
    be.gather_rows(host, T(ids), T(mask), out=out, accumulate=True)
    np.testing.assert_array_equal(out.cpu().numpy(),
                                  1 + orc.gather_rows(host.float().numpy(), ids, mask))
    # destination in the source's own precision (fp16 feature files stay fp16)
    got16 = be.gather_rows(host, T(ids), T(mask), out_dtype=torch.float16)
    assert got16.dtype == torch.float16
    np.testing.assert_array_equal(got16.float().cpu().numpy(), orc.gather_rows(host.float().numpy(), ids, mask))
    m = rng.integers(-1, 99, size=1000)
    np.testing.assert_array_equal(be.lookup(T(m), T(ids), 3).cpu().numpy(), m[ids + 3])


@pytest.mark.parametrize("n", [1, 2, 3, 257, 1024, 1025, 5800, 10_000, 1 << 14, (1 << 14) + 1, 1 << 15, (1 << 15) + 1, 1 << 17, (1 << 17) + 3, 200_003, 2_000_000, 5_000_001])
def test_quantile_threshold_by_selection_equals_the_sort(n):
    """hc_quantile_threshold_ws (radix select of the two order statistics + the interpolation: one launch by one
    block up to 2^17 scores, the whole chip above) gives the bits of the sorted spelling -- which is
    torch.quantile's rule, pinned on the CPU side -- for rates over [0, 1], negative scores, ties, infinities."""
    from hiscache.util import quantile_threshold
    rng = np.random.default_rng(n)
    cases = [rng.standard_normal(n), np.abs(rng.standard_normal(n)) * np.exp(rng.normal(-3, 1.5, size=n)),
             rng.integers(0, 4, size=n).astype(np.float64), np.full(n, 0.25)]
    # scores that share most of their bits: two neighbouring floats, and a range of 2^13 and of 2^5 neighbours
    one = np.float32(1.0)
    cases.append(np.where(rng.random(n) < 0.3, one, np.nextafter(one, np.float32(2))).astype(np.float32))
    for span in (1 << 13, 1 << 5):
        cases.append((one.view(np.uint32) + rng.integers(0, span, size=n).astype(np.uint32)).view(np.float32))
    if n > 3:
        wild = rng.standard_normal(n)
        wild[:2] = [np.inf, -np.inf]
        cases.append(wild)
    for s in cases:
        s32 = s.astype(np.float32)
        dev = torch.from_numpy(s32).to(DEV)
        for rate in (0.0, 0.1, 0.5, 0.7, 0.9, 0.999, 1.0) if n <= 1 << 18 else (0.0, 0.5, 0.999999, 1.0):
            got = quantile_threshold(dev, rate)
            want = quantile_threshold(torch.from_numpy(s32), rate)
            assert got.is_cuda and got.shape == (1,)
            np.testing.assert_array_equal(got.cpu().numpy().view(np.uint32), want.numpy().view(np.uint32),
                                          err_msg=f"n={n} rate={rate}")
    if n > 8:
        # a NaN score of either sign makes the threshold NaN, as torch.quantile does
        # (/root/reference/hiscache/history_cache.py:211): `score < thres` then admits nothing
        s32 = rng.standard_normal(n).astype(np.float32)
        s32[1], s32[5] = np.float32(np.nan), -np.float32(np.nan)
        dev = torch.from_numpy(s32).to(DEV)
        for rate in (0.0, 0.3, 0.5, 1.0):
            got = quantile_threshold(dev, rate).cpu().numpy()
            want = quantile_threshold(torch.from_numpy(s32), rate).numpy()
            ref = torch.quantile(torch.from_numpy(s32), rate).numpy()
            assert np.isnan(got[0]) and np.isnan(want[0]) and np.isnan(ref), f"n={n} rate={rate}"
            assert int((dev < torch.from_numpy(got).to(DEV)).sum()) == 0


def test_quantile_entry_points_state_their_limits():
    """The one-block entry point refuses more scores than hc_quantile_max_scores() with HC_EUNSUPPORTED and
    launches nothing; the workspace variant refuses a workspace that is too small."""
    import hiscache_backend as be
    lib = be.load_library()
    limit = int(lib.hc_quantile_max_scores())
    assert limit == 1 << 17
    score = torch.rand(limit + 1, device=DEV)
    out = torch.full((1,), -7.0, device=DEV)
    rc = lib.hc_quantile_threshold(be._ptr(score), limit + 1, 3, 4, 0.25, 0.75, be._ptr(out), be._stream())
    assert rc == 5                                   # HC_EUNSUPPORTED
    need = int(lib.hc_quantile_workspace_bytes(limit + 1))
    assert need > 0 and int(lib.hc_quantile_workspace_bytes(1000)) == 0
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    rc = lib.hc_quantile_threshold_ws(be._ptr(score), limit + 1, 3, 4, 0.25, 0.75, be._ptr(out), be._ptr(ws), need - 1,
                                      be._stream())
    assert rc != 0
    torch.cuda.synchronize()
    assert float(out) == -7.0
    rc = lib.hc_quantile_threshold_ws(be._ptr(score), limit + 1, 3, 4, 0.25, 0.75, be._ptr(out), be._ptr(ws), need,
                                      be._stream())
    assert rc == 0
    srt = torch.sort(score).values
    want = srt[3] + (srt[4] - srt[3]) * 0.25
    assert float(out) == float(want)
