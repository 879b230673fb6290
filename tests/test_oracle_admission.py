"""Pins the CPU oracle's used-mask, admission and cache-policy routines against brute-force models,
library routines and invariants.  No GPU."""
import numpy as np
import pytest
import torch

from helpers import layered_batch, random_csr


# ----------------------------------------------------------------------------- used masks
def brute_used_masks(ptr, idx, hmap, n_all, n_seed, L):
    """Frontier expansion, level by level, in plain Python (the rule of
    /root/reference/src/cpp/src/grad_check.cu:79-100)."""
    masks = [set() for _ in range(L + 1)]
    masks[L] = set(range(n_seed))
    rows = len(ptr) - 1
    for i in range(L):
        use_in, use_out = masks[L - i], masks[L - 1 - i]
        for r in sorted(use_in):
            if r >= rows:
                continue
            if i == 1 and hmap is not None and hmap[r] != -1:
                continue
            use_out.add(r)
            use_out.update(int(v) for v in idx[ptr[r]:ptr[r + 1]])
    out = np.zeros((L + 1, n_all), bool)
    for k in range(L + 1):
        out[k, sorted(masks[k])] = True
    return out


def reference_invalidate(cached, useful, num1, num2, ptr, idx):
    """The reference's own CPU snippet (/root/reference/test/test_cache.py:165-174), restated:
    a useful, un-cached row makes its neighbours useful (it has no self-mark)."""
    useful2 = np.zeros(num2, bool)
    for i in range(num1):
        if not cached[i] and useful[i]:
            useful2[idx[ptr[i]:ptr[i + 1]]] = True
    return useful2


@pytest.mark.parametrize("seed,L,fanout", [(0, 2, [4, 3]), (1, 3, [5, 3, 2]), (2, 1, [6]), (3, 3, [2, 2, 2])])
def test_count_history_brute_force(orc, seed, L, fanout):
    rng = np.random.default_rng(seed)
    b = layered_batch(rng, 400, 12, fanout)
    ptr, idx, nnl = b["ptr"], b["idx"], b["num_node_in_layer"]
    n_all, n_seed, n1 = int(nnl[-1]), int(nnl[0]), int(nnl[1])
    hmap = np.full(n1, -1, np.int64)
    hmap[rng.random(n1) < 0.4] = 7
    got = np.stack(orc.count_history_reconstruct(ptr, idx, hmap, n_all, n_seed, L))
    np.testing.assert_array_equal(got, brute_used_masks(ptr, idx, hmap, n_all, n_seed, L))
    # no history: level k holds exactly the nodes within L-k hops of the seeds
    nohist = np.stack(orc.count_history_reconstruct(ptr, idx, None, n_all, n_seed, L))
    for k in range(L + 1):
        expect = np.zeros(n_all, bool)
        expect[:nnl[L - k]] = True
        np.testing.assert_array_equal(nohist[k], expect)
    # pruning only ever removes nodes
    assert not (got & ~nohist).any()


def test_count_history_against_reference_snippet(orc):
    """Chain the reference's invalidate() over the layers; add the self-mark the kernel has
    (grad_check.cu:92-94) and the kernel's rule that history is consulted on the second pass only."""
    rng = np.random.default_rng(4)
    L = 3
    b = layered_batch(rng, 600, 10, [4, 3, 2])
    ptr, idx, nnl = b["ptr"], b["idx"], b["num_node_in_layer"]
    n_all, n_seed, n1 = int(nnl[-1]), int(nnl[0]), int(nnl[1])
    hmap = np.full(n1, -1, np.int64)
    hmap[rng.random(n1) < 0.5] = 3
    got = np.stack(orc.count_history_reconstruct(ptr, idx, hmap, n_all, n_seed, L))
    rows = len(ptr) - 1
    useful = np.zeros(n_all, bool)
    useful[:n_seed] = True
    for i in range(L):
        cached = np.zeros(rows, bool)
        if i == 1:
            cached[:n1] = hmap != -1
        nxt = reference_invalidate(cached, useful, rows, n_all, ptr, idx)
        nxt[:rows] |= useful[:rows] & ~cached      # the self-mark
        useful = nxt
        np.testing.assert_array_equal(got[L - 1 - i], useful)


def test_count_history_all_cached_prunes_subtrees(orc):
    rng = np.random.default_rng(5)
    b = layered_batch(rng, 500, 8, [3, 3, 3])
    ptr, idx, nnl = b["ptr"], b["idx"], b["num_node_in_layer"]
    n_all, n_seed, n1 = int(nnl[-1]), int(nnl[0]), int(nnl[1])
    hmap = np.zeros(n1, np.int64)                  # every 1-hop row is cached
    got = orc.count_history_reconstruct(ptr, idx, hmap, n_all, n_seed, 3)
    assert got[3][:n_seed].all() and not got[3][n_seed:].any()
    assert got[2][:n1].all() and not got[2][n1:].any()
    assert not got[1].any() and not got[0].any()   # nothing below a cached row is needed


# ----------------------------------------------------------------------------- scores
def test_row_scores_close_to_library_norms(orc):
    rng = np.random.default_rng(6)
    for F in (1, 3, 64, 255, 256, 300, 1024):
        g = (rng.standard_normal((17, F)) * 10.0 ** rng.integers(-4, 3, size=(17, 1))).astype(np.float32)
        l2 = orc.row_scores(g, orc.NORM_L2)
        l1 = orc.row_scores(g, orc.NORM_L1)
        np.testing.assert_allclose(l2, np.linalg.norm(g.astype(np.float64), axis=1), rtol=2e-6)
        np.testing.assert_allclose(l1, np.abs(g.astype(np.float64)).sum(1), rtol=2e-6)
        np.testing.assert_allclose(l2, torch.from_numpy(g).norm(dim=1).numpy(), rtol=2e-6)


def test_row_score_summation_order(orc):
    """The documented order: lane (e/4)%64 folds its elements with fma in increasing e, then a
    butterfly 32,16,...,1 -- written out independently with NumPy float32 scalars."""
    rng = np.random.default_rng(7)
    F = 600
    row = rng.standard_normal(F).astype(np.float32)
    acc = [np.float32(0)] * 64
    for e in range(F):
        l = (e // 4) % 64
        acc[l] = np.float32(np.float64(row[e]) * np.float64(row[e]) + np.float64(acc[l]))  # fma: one rounding
    for d in (32, 16, 8, 4, 2, 1):
        acc = [np.float32(acc[l] + acc[l ^ d]) for l in range(64)]
    expect = np.sqrt(acc[0], dtype=np.float32)
    assert orc.row_scores(row[None, :], orc.NORM_L2)[0] == expect


def test_half_conversions_match_numpy_and_torch(orc):
    rng = np.random.default_rng(8)
    x = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, size=4000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -14, 6.1e-5, 5.96e-8, np.inf, -np.inf], np.float32),
        np.float32(1.0) + np.arange(-3, 4, dtype=np.float32) * np.float32(2.0 ** -11),   # ties
    ]).astype(np.float32)
    np.testing.assert_array_equal(orc.f32_to_f16_bits(x), x.astype(np.float16).view(np.uint16))
    bf = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(orc.f32_to_bf16_bits(x), bf)


# ----------------------------------------------------------------------------- ring admission
class DictRing:
    """Ring-buffer cache as dictionaries, slots handed out in row order
    (the insert of /root/reference/src/cpp/src/grad_check.cu:22-45)."""

    def __init__(self, cap, header=0):
        self.cap, self.header = cap, header
        self.slot_owner = {}      # slot -> node      (history_to_full)
        self.node_slot = {}       # node -> slot      (full_to_history)
        self.checkin = {}
        self.rows = {}

    def insert(self, node, row, it):
        s = self.header
        self.header = 0 if s >= self.cap - 1 else s + 1
        old = self.slot_owner.get(s)
        if old is not None and self.node_slot.get(old) == s:
            del self.node_slot[old]
        self.node_slot[node] = s
        self.slot_owner[s] = node
        self.checkin[s] = it
        self.rows[s] = row
        return s


def check_ring(model, buffer_all, h2f, f2h, checkin, header):
    assert header[0] == model.header
    for s in range(model.cap):
        assert h2f[s] == model.slot_owner.get(s, -1)
        assert checkin[s] == model.checkin.get(s, -1)
        if s in model.rows:
            np.testing.assert_array_equal(buffer_all[s], model.rows[s])
    expect = np.full(len(f2h), -1, np.int64)
    for n, s in model.node_slot.items():
        expect[n] = s
    np.testing.assert_array_equal(f2h, expect)
    # invariants: live slots point back at their owner; no node owns two live slots
    live = [(n, s) for n, s in model.node_slot.items()]
    assert len({s for _, s in live}) == len(live)
    for n, s in live:
        assert h2f[s] == n


@pytest.mark.parametrize("cap", [8, 37, 400])
def test_record_history_ring_model(orc, cap):
    rng = np.random.default_rng(9)
    N, hs = 300, 5
    buffer_all = np.zeros((cap, hs), np.float32)
    h2f = np.full(cap, -1, np.int64)
    f2h = np.full(N, -1, np.int64)
    checkin = np.full(cap, -1, np.int64)
    header = np.zeros(1, np.int64)
    model = DictRing(cap)
    for it in range(6):
        M = int(rng.integers(5, 60))
        sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int64)
        new = rng.standard_normal((M, hs)).astype(np.float32)
        score = rng.random(M).astype(np.float32)
        thres = np.float32(np.sort(score)[int(0.7 * (M - 1))])       # some scores equal thres exactly
        used = rng.random(M) < 0.8
        sub2hist = f2h[sub_to_full].copy()
        sub2hist[: M // 5] = -1                                       # seeds are forced to -1
        mask = orc.record_history(new, buffer_all, used, sub_to_full, sub2hist, h2f, f2h, header, score,
                                  thres, checkin, it)
        expect_mask = (sub2hist == -1) & ~((thres != 0) & (score > thres)) & used
        np.testing.assert_array_equal(mask, expect_mask)
        assert mask[score == thres].sum() == ((sub2hist == -1) & used)[score == thres].sum()  # equality admitted
        for r in np.flatnonzero(expect_mask):
            model.insert(int(sub_to_full[r]), new[r], it)
        check_ring(model, buffer_all, h2f, f2h, checkin, header)


def test_record_history_zero_threshold_admits_everything(orc):
    M, cap, hs = 10, 16, 3
    args = dict(buffer_all=np.zeros((cap, hs), np.float32), h2f=np.full(cap, -1, np.int64),
                f2h=np.full(50, -1, np.int64), checkin=np.full(cap, -1, np.int64), header=np.zeros(1, np.int64))
    mask = orc.record_history(np.ones((M, hs), np.float32), args["buffer_all"], np.ones(M, bool),
                              np.arange(M), np.full(M, -1), args["h2f"], args["f2h"], args["header"],
                              np.full(M, 5.0, np.float32), np.float32(0.0), args["checkin"], 3)
    assert mask.all() and args["header"][0] == M       # thres == 0 disables the score test (grad_check.cu:18)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_grad_check_equals_scores_plus_ring(orc, dtype):
    """The fused pass equals row_scores followed by the dict ring model, for both comparison kinds,
    with staleness ages, and with a reduced-precision table."""
    rng = np.random.default_rng(10)
    N, F, cap, M = 500, 24, 64, 150
    code = {"f32": orc.DT_F32, "f16": orc.DT_F16, "bf16": orc.DT_BF16}[dtype]
    table = np.zeros((cap, F), np.float32 if dtype == "f32" else np.uint16)
    f2s = np.full(N, -1, np.int64)
    s2f = np.full(cap, -1, np.int64)
    checkin = np.full(cap, -1, np.int64)
    header = np.array([cap - 7], np.int64)            # forces a wrap
    model = DictRing(cap, header=cap - 7)
    for it, cmp_kind in enumerate([orc.CMP_LT, orc.CMP_NOT_GT, orc.CMP_LT]):
        sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int64)
        grad = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
        emb = rng.standard_normal((M, F)).astype(np.float32)
        slot = f2s[sub_to_full].copy()
        age = rng.integers(0, 21, size=M).astype(np.int32)
        used = rng.random(M) < 0.9
        score = orc.row_scores(grad)
        thres = float(np.sort(score)[M // 2])          # one score equals the threshold
        mask, sc, slots = orc.grad_check(grad, emb, slot, age, used, sub_to_full, thres, 10, orc.NORM_L2,
                                         cmp_kind, table, code, f2s, s2f, checkin, header, it)
        np.testing.assert_array_equal(sc, score)
        passed = score < np.float32(thres) if cmp_kind == orc.CMP_LT else ~((thres != 0) & (score > np.float32(thres)))
        expect = used & passed & ((slot == -1) | (age >= 10))
        np.testing.assert_array_equal(mask, expect)
        for r in np.flatnonzero(expect):
            row = emb[r]
            if dtype == "f16":
                row = emb[r].astype(np.float16).view(np.uint16)
            elif dtype == "bf16":
                row = torch.from_numpy(emb[r]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
            s = model.insert(int(sub_to_full[r]), row, it)
            assert slots[r] == s
        assert (slots[~expect] == -1).all()
        check_ring(model, table, s2f, f2s, checkin, header)


def test_grad_check_more_admitted_than_capacity(orc):
    rng = np.random.default_rng(11)
    N, F, cap, M = 200, 8, 10, 45
    table = np.zeros((cap, F), np.float32)
    f2s, s2f = np.full(N, -1, np.int64), np.full(cap, -1, np.int64)
    checkin, header = np.full(cap, -1, np.int64), np.array([3], np.int64)
    model = DictRing(cap, header=3)
    sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int64)
    emb = rng.standard_normal((M, F)).astype(np.float32)
    mask, _, _ = orc.grad_check(None, emb, np.full(M, -1), None, None, sub_to_full, 1.0, 0, orc.NORM_L2,
                                orc.CMP_LT, table, orc.DT_F32, f2s, s2f, checkin, header, 5,
                                score_in=np.zeros(M, np.float32))
    assert mask.all()
    for r in range(M):
        model.insert(int(sub_to_full[r]), emb[r], 5)
    check_ring(model, table, s2f, f2s, checkin, header)
    assert (f2s != -1).sum() == cap


def test_grad_check_large_block_with_used_mask(orc):
    """A block large enough that a converted copy of the used mask would be recycled by the allocator
    if the wrapper let go of it before the C call: the mask equals the numpy predicate."""
    rng = np.random.default_rng(13)
    N, F, cap, M = 40000, 16, 700, 8000
    table = np.zeros((cap, F), np.float32)
    f2s, s2f = np.full(N, -1, np.int64), np.full(cap, -1, np.int64)
    checkin, header = np.full(cap, -1, np.int64), np.array([5], np.int64)
    for it in range(3):
        sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int32)     # converted by the wrapper
        grad = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
        emb = rng.standard_normal((M, F)).astype(np.float32)
        slot = f2s[sub_to_full].astype(np.int32)                               # converted by the wrapper
        age = rng.integers(0, 21, size=M).astype(np.int32)
        used = rng.random(M) < 0.9
        score = orc.row_scores(grad)
        thres = float(np.sort(score)[M // 3])
        mask, _, _ = orc.grad_check(grad, emb, slot, age, used, sub_to_full, thres, 10, orc.NORM_L2, orc.CMP_LT,
                                    table, orc.DT_F32, f2s, s2f, checkin, header, it)
        expect = used & (score < np.float32(thres)) & ((slot == -1) | (age >= 10))
        np.testing.assert_array_equal(mask, expect)


def test_multithreaded_admission_equals_the_sequential_one(orc):
    """The OpenMP admission that the benchmark times as its CPU baseline: scores, mask, maps, header and
    fp16 table bit for bit equal to the sequential statement, across a ring wrap and with stale rows
    re-admitted; its fp32 -> fp16 rounding equals NumPy's."""
    from oracle import hc_cpu_mt as mt
    rng = np.random.default_rng(14)
    v = np.concatenate([rng.standard_normal(3000).astype(np.float32) * np.float32(10) ** rng.integers(-9, 5, size=3000).astype(np.float32),
                        np.array([0, -0.0, 65504, 65519.99, 65520, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                                  2.0 ** -14, 2.0 ** -14 * 0.9999, 5.96e-8, 3e-8], np.float32)])
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(mt.f32_to_f16_bits(v), v.astype(np.float16).view(np.uint16))
        for hw in (False, True):                       # portable build and the FMA / F16C build
            np.testing.assert_array_equal(mt.convert_row(v, hw), v.astype(np.float16).view(np.uint16))
    for width in (1, 5, 64, 255, 256, 300, 768):
        g = (rng.standard_normal((50, width)) * np.exp(rng.normal(-3, 1.5, size=(50, 1)))).astype(np.float32)
        for hw in (False, True):
            np.testing.assert_array_equal(mt.score_rows(g, hw), orc.row_scores(g))
    N, F, cap, M = 40000, 64, 9000, 8000
    ref = dict(table=np.zeros((cap, F), np.uint16), f2s=np.full(N, -1, np.int64), s2f=np.full(cap, -1, np.int64),
               checkin=np.full(cap, -1, np.int64), header=np.array([cap - 100], np.int64))
    got = {k: a.copy() for k, a in ref.items()}
    readmitted = 0
    for it in range(5):
        nodes = rng.choice(N, size=M, replace=False).astype(np.int64)
        grad = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
        emb = rng.standard_normal((M, F)).astype(np.float32)
        slot = ref["f2s"][nodes].copy()
        age = rng.integers(0, 21, size=M).astype(np.int32)
        thres = float(np.sort(orc.row_scores(grad))[M // 4])
        rmask, rscore, _ = orc.grad_check(grad, emb, slot, age, None, nodes, thres, 10, orc.NORM_L2, orc.CMP_LT,
                                          ref["table"], orc.DT_F16, ref["f2s"], ref["s2f"], ref["checkin"],
                                          ref["header"], it)
        mask, score = mt.grad_check_f16(grad, emb, slot, age, nodes, thres, 10, got["table"], got["f2s"], got["s2f"],
                                        got["checkin"], got["header"], it)
        np.testing.assert_array_equal(mask, rmask)
        np.testing.assert_array_equal(score, rscore)
        for k in ref:
            np.testing.assert_array_equal(got[k], ref[k], err_msg=k)
        readmitted += int(((slot != -1) & rmask).sum())
    assert readmitted > 100 and ref["header"][0] < cap - 100          # stale rows came back, the ring wrapped
    small = np.zeros((10, F), np.uint16)
    with pytest.raises(ValueError):                                    # more admitted rows than slots
        mt.grad_check_f16(grad, emb, np.full(M, -1), None, nodes, 1e9, 10, small, got["f2s"], np.full(10, -1, np.int64),
                          None, np.zeros(1, np.int64), 9)


# ----------------------------------------------------------------------------- thresholds
def test_quantile_threshold_matches_torch_quantile():
    from oracle import host_model
    rng = np.random.default_rng(12)
    worst = 0
    for n in (1, 2, 3, 10, 101, 1000, 4097):
        for rate in (0.0, 0.1, 0.5, 0.9, 0.999, 1.0):
            s = np.exp(rng.normal(-3, 1.5, size=n)).astype(np.float32)
            mine = host_model.quantile_threshold(s, rate)
            ref = torch.quantile(torch.from_numpy(s), rate).numpy()
            ulp = abs(int(np.float32(mine).view(np.int32)) - int(np.float32(ref).view(np.int32)))
            worst = max(worst, ulp)
    assert worst <= 2, worst


def test_quantile_threshold_is_nan_when_a_score_is_nan():
    """torch.quantile answers NaN when any score is NaN (the reference then admits nothing,
    hiscache/history_cache.py:211-215); the restatement and the package's host spelling do the same."""
    from hiscache.util import quantile_threshold as pkg_quantile
    from oracle import host_model
    s = np.random.default_rng(3).standard_normal(500).astype(np.float32)
    s[17] = np.nan
    for rate in (0.0, 0.5, 1.0):
        assert np.isnan(torch.quantile(torch.from_numpy(s), rate).numpy())
        assert np.isnan(host_model.quantile_threshold(s, rate))
        t = pkg_quantile(torch.from_numpy(s), rate)
        assert np.isnan(t.numpy()[0]) and int((torch.from_numpy(s) < t).sum()) == 0


def test_quantile_threshold_gives_torch_quantiles_admission_mask():
    """The reference thresholds with torch.quantile (hiscache/history_cache.py:211-215).  Over 1 200
    seeded batches at the 1-hop sizes of the plumbing and papers100M-shaped configurations (scores
    with the lognormal spread of gradient norms, rates 0.5 / 0.7 / 0.9) the mask ``score < threshold``
    from the build's threshold (host statement and the package's own function) is compared with the
    mask from torch.quantile on the same scores: a row may only differ when its score lies within
    2 ulp of torch's threshold; such rows are counted and reported."""
    from hiscache.util import quantile_threshold as pkg_quantile
    from oracle import host_model
    rng = np.random.default_rng(2111)
    knife, differ, same_bits = 0, 0, 0
    sizes = [11_000, 5_544, 10_873, 16_000, 7, 1_000]
    n_batches = 1200
    for it in range(n_batches):
        n = sizes[it % len(sizes)] + int(rng.integers(0, 50))
        rate = (0.5, 0.7, 0.9)[it % 3]
        s = np.exp(rng.normal(-3, 1.5, size=n)).astype(np.float32)
        if it % 7 == 0:
            s[rng.integers(0, n, size=n // 4)] = s[0]            # many equal scores around the threshold
        ref = torch.quantile(torch.from_numpy(s), rate).numpy().astype(np.float32)
        mine = np.float32(host_model.quantile_threshold(s, rate))
        pkg = pkg_quantile(torch.from_numpy(s), rate).numpy().astype(np.float32).reshape(())
        assert pkg.view(np.int32) == mine.view(np.int32)          # host statement and package function agree
        same_bits += int(mine.view(np.int32) == ref.view(np.int32))
        # scores within 2 ulp of torch's threshold (positive floats: ordered like their bit patterns)
        near = np.abs(s.view(np.int32).astype(np.int64) - int(ref.view(np.int32))) <= 2
        knife += int(near.sum())
        diff = (s < mine) != (s < ref)
        differ += int(diff.sum())
        assert not (diff & ~near).any(), "a row outside the 2-ulp band changed sides (batch %d)" % it
    print("quantile masks: %d batches, threshold bit-identical to torch.quantile in %d; %d rows within 2 ulp of "
          "the threshold, %d of them on the other side" % (n_batches, same_bits, knife, differ))
    assert same_bits >= 0.9 * n_batches


# ----------------------------------------------------------------------------- structure score
def random_forest_batch(rng, n_seed, depth, max_children):
    """A layered batch whose rows form a forest: every node is the neighbour of exactly one row, so
    every node is reached along exactly one path from a seed, at most ``depth`` hops long."""
    ptr, idx = [0], []
    level = list(range(n_seed))
    n_nodes = n_seed
    parent_deg_product = {v: 1 for v in level}        # product of the degrees of a node's ancestors
    for d in range(depth):
        nxt = []
        for u in level:                                # rows are numbered in node order, level by level
            c = int(rng.integers(0, max_children + 1))
            kids = list(range(n_nodes, n_nodes + c))
            n_nodes += c
            idx.extend(kids)
            ptr.append(len(idx))
            for k in kids:
                parent_deg_product[k] = parent_deg_product[u] * c
            nxt.extend(kids)
        level = nxt
    return np.asarray(ptr, np.int64), np.asarray(idx, np.int64), n_nodes, parent_deg_product


@pytest.mark.parametrize("seed,n_seed,depth,kids", [(1, 5, 3, 4), (2, 40, 2, 7), (3, 1, 4, 3), (4, 30, 3, 6)])
def test_structure_score_on_forests_has_the_references_only_possible_result(orc, seed, n_seed, depth, kids):
    """get_graph_structure_score (src/cpp/src/grad_check.cu:132-163) reads and writes its output
    across warps inside one pass, so in general its result depends on scheduling.  On a forest of
    depth <= num_layer every node receives exactly one offer, whatever the interleaving: the product
    of the degrees of its ancestors.  There the reference has one possible answer and the
    level-synchronous statement must give it; seeds keep 1, unreached ids keep 0."""
    rng = np.random.default_rng(seed)
    ptr, idx, n_nodes, want = random_forest_batch(rng, n_seed, depth, kids)
    # shuffle the neighbour ids' numbering beyond the rows so that node order is not level order
    n_rows = len(ptr) - 1
    perm = np.arange(n_nodes + 3)                     # three extra ids that nothing reaches
    tail = perm[n_rows:].copy()
    rng.shuffle(tail)
    perm[n_rows:] = tail
    idx2 = perm[idx]
    got = orc.get_graph_structure_score(ptr, idx2, n_nodes + 3, n_seed, depth)
    expect = np.zeros(n_nodes + 3, np.int64)
    for v, prod in want.items():
        expect[perm[v]] = prod
    np.testing.assert_array_equal(got, expect)
    # more passes than levels change nothing; fewer passes reach fewer levels
    np.testing.assert_array_equal(orc.get_graph_structure_score(ptr, idx2, n_nodes + 3, n_seed, depth + 2), expect)


# ----------------------------------------------------------------------------- cache policy
class DictCache:
    """HistoryCache.update_history as a dictionary model: embeddings appended at `header`,
    overlapped feature slots dropped, overwritten embedding slots un-mapped
    (/root/reference/hiscache/history_cache.py:216-254)."""

    def __init__(self, st):
        self.emb_slot = {}                       # node -> embedding slot
        self.slot_owner = {}                     # embedding slot -> node (may be stale)
        self.feat_slot = {int(f) - st.N: i for i, f in enumerate(st.feat2full.tolist()) if f >= 0}
        self.H, self.Fin = st.H, st.Fin
        self.header = 0

    def append(self, nodes):
        h, n = self.header, len(nodes)
        lo, hi = h * self.H // self.Fin, -(-(h + n) * self.H // self.Fin)
        self.feat_slot = {k: v for k, v in self.feat_slot.items() if not (lo <= v < hi)}
        for s in range(h, h + n):
            old = self.slot_owner.get(s)
            if old is not None and h <= self.emb_slot.get(old, -1) < h + n:
                del self.emb_slot[old]
        for k, node in enumerate(nodes):
            self.emb_slot[node] = h + k
            self.slot_owner[h + k] = node
        self.header += n


def test_update_history_dict_model(orc):
    from oracle import host_model
    rng = np.random.default_rng(13)
    N, Fin, H = 400, 8, 12
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    hot = rng.permutation(N).astype(np.int64)
    st = host_model.new_cache_state(N, Fin, H, 24 * 60, hot, feats)       # 180 feature slots, 120 embedding slots
    model = DictCache(st)
    for it in range(1, 9):
        M = int(rng.integers(20, 60))
        nodes = torch.from_numpy(rng.choice(N, size=M, replace=False).astype(np.int64))
        sub2embed = st.full2embed[nodes]
        emb = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32))
        score = torch.from_numpy(np.exp(rng.normal(-3, 1.5, size=M)).astype(np.float32))
        if it % 4 == 0:
            model.header = 0                                              # staleness refresh
        header_before = 0 if it % 4 == 0 else st.header
        mask, thres = host_model.update_history(st, nodes, sub2embed, emb, score, 0.6, 4, it)
        expect = (score.numpy() < thres) & (sub2embed.numpy() == -1)
        np.testing.assert_array_equal(mask.numpy(), expect)
        model.append([int(v) for v in nodes.numpy()[expect]])
        assert st.header == model.header == header_before + int(expect.sum())
        f2e = st.full2embed.numpy()
        exp_e = np.full(N, -1, np.int64)
        for n_, s_ in model.emb_slot.items():
            exp_e[n_] = s_
        np.testing.assert_array_equal(f2e[:N], exp_e)
        exp_f = np.full(N, -1, np.int64)
        for n_, s_ in model.feat_slot.items():
            exp_f[n_] = s_
        np.testing.assert_array_equal(f2e[N:2 * N], exp_f)
        assert f2e[2 * N] == -1                                           # the sentinel entry is never set
        # stored rows are the admitted embeddings, in row order
        np.testing.assert_array_equal(
            st.buffer.view(-1, H)[header_before:st.header].numpy(), emb.numpy()[expect])


def test_lookup_and_load_closed_form(orc):
    """batch.x[i] equals the node's feature row for every node still needed, whether it came from
    the feature cache or from host memory; other rows are zero unless feature-cached."""
    from oracle import host_model
    from types import SimpleNamespace
    rng = np.random.default_rng(14)
    N, Fin, H = 500, 6, 10
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    st = host_model.new_cache_state(N, Fin, H, 30 * 40, rng.permutation(N).astype(np.int64), feats)
    b = layered_batch(rng, N, 10, [4, 3])
    batch = SimpleNamespace(ptr=torch.from_numpy(b["ptr"]), idx=torch.from_numpy(b["idx"]),
                            sub_to_full=torch.from_numpy(b["sub_to_full"]),
                            num_node_in_layer=torch.from_numpy(b["num_node_in_layer"]),
                            y=torch.zeros(10, dtype=torch.int64))
    n1 = int(b["num_node_in_layer"][1])
    # cache a few 1-hop embeddings first
    nodes = batch.sub_to_full[:n1]
    emb = torch.from_numpy(rng.standard_normal((n1, H)).astype(np.float32))
    score = torch.from_numpy(rng.random(n1).astype(np.float32))
    host_model.update_history(st, nodes, st.full2embed[nodes], emb, score, 0.5, 100, 1)
    out = host_model.lookup_and_load(st, batch, 2, feats)
    full = feats[batch.sub_to_full]
    needed = out.used_masks[0]
    hit = out.sub2feat != -1
    np.testing.assert_array_equal(out.x[needed | hit].numpy(), full[needed | hit].numpy())
    assert (out.x[~(needed | hit)] == 0).all()
    cached = out.sub2embed != -1
    assert cached.any() and (~needed).any()
    np.testing.assert_array_equal(out.cached_embedding[cached].numpy(),
                                  st.buffer.view(-1, H)[out.sub2embed[cached]].numpy())


def test_evict_by_staleness_rule():
    from oracle import host_model
    checkin = torch.tensor([-1, 0, 3, 5, 7, 10])
    h2f = torch.tensor([-1, 11, 12, 13, 14, 15])
    f2h = torch.full((20,), -1, dtype=torch.int64)
    f2h[h2f[1:]] = torch.arange(1, 6)
    host_model.evict_by_staleness(checkin, h2f, f2h, glb_iter=10, staleness_thres=5)
    assert checkin.tolist() == [-1, -1, -1, -1, 7, 10]          # -1 < checkin <= 5 evicted
    assert h2f.tolist() == [-1, -1, -1, -1, 14, 15]
    assert (f2h[[11, 12, 13]] == -1).all() and f2h[14] == 4 and f2h[15] == 5


def test_small_helpers(orc):
    rng = np.random.default_rng(15)
    arr = rng.integers(0, 6, size=1000)
    np.testing.assert_array_equal(orc.count_num(arr, 5)[1:], np.bincount(arr, minlength=6)[1:])
    assert orc.count_num(arr, 5)[0] == 0                        # value 0 is skipped (grad_check.cu:169)
    # structure score on a path graph 0 -> 1 -> 2 with a branch
    ptr = np.array([0, 2, 3, 3, 3]); idx = np.array([1, 2, 3])
    s = orc.get_graph_structure_score(ptr, idx, 4, 1, 2)
    assert s.tolist() == [1, 2, 2, 2]
    t = rng.standard_normal((7, 3)).astype(np.float32)
    got = orc.gather_rows(t, np.array([0, -1, 3]), np.array([True, True, False]))
    np.testing.assert_array_equal(got, np.stack([t[0], t[6], np.zeros(3, np.float32)]))


def typed_csr_by_stable_sort(ptr, idx, rel, K, R, n_src, used=None):
    """(row, relation) grouping stated with numpy: keep-filter, then a stable sort by row*K + relation."""
    E = min(len(idx), len(rel))
    row_of = np.searchsorted(ptr[1:R + 1], np.arange(E), side="right")
    keep = (row_of < R) & (rel[:E] >= 0) & (rel[:E] < K) & (idx[:E] >= 0) & (idx[:E] < n_src)
    if used is not None:
        keep &= used[np.clip(idx[:E], 0, n_src - 1)]
    key = row_of[keep] * K + rel[:E][keep]
    order = np.argsort(key, kind="stable")
    cnt = np.bincount(key, minlength=R * K)[:R * K]
    ptr2 = np.concatenate([[0], np.cumsum(cnt)])
    return ptr2, idx[:E][keep][order], cnt.reshape(R, K), np.diff(ptr)[:R]


@pytest.mark.parametrize("K,with_mask,short_types", [(5, True, False), (1, False, False), (64, True, True),
                                                      (7, False, True)])
def test_typed_csr_equals_stable_sort(orc, K, with_mask, short_types):
    from helpers import random_csr
    rng = np.random.default_rng(40 + K)
    R, N = 120, 90
    ptr, idx = random_csr(rng, R + 30, N, 150, hub=3)          # some rows longer than 64 edges
    idx = idx.copy()
    idx[rng.random(len(idx)) < 0.02] = N + 5                    # sources outside the range are dropped
    rel = rng.integers(-1, K + 1, size=len(idx))                # -1 and K are dropped
    if short_types:
        rel = rel[: int(ptr[R - 10])]                           # the last rows have no relation entries
    used = (rng.random(N) < 0.7) if with_mask else None
    want = typed_csr_by_stable_sort(ptr, idx, rel, K, R, N, used)
    got = orc.typed_csr(ptr, idx, rel, K, R, N, used)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g, w)
    # no rows: a single zero offset
    p2, i2, c, d = orc.typed_csr(ptr, idx, rel, K, 0, N, used)
    assert p2.tolist() == [0] and i2.size == 0 and c.size == 0 and d.size == 0
    # edge weights: one loop over the groups; the weighted sums of a row's groups add up to the row's mean
    # over all its edges restricted to the kept ones
    ptr2, idx2, cnt, deg = got
    wts = orc.typed_csr_weights(ptr2, deg, K)
    assert wts.dtype == np.float32 and len(wts) == ptr2[-1]
    for v in range(R * K):
        r = v // K
        assert (wts[ptr2[v]:ptr2[v + 1]] == np.float32(1.0) / np.float32(max(int(deg[r]), 1))).all()
    x = rng.standard_normal(N + 6)
    for r in (0, R // 2, R - 1):
        kept = idx2[ptr2[r * K]:ptr2[(r + 1) * K]]
        want_mean = x[kept].sum() / max(int(deg[r]), 1)
        got_mean = sum(float(wts[e]) * x[idx2[e]] for e in range(ptr2[r * K], ptr2[(r + 1) * K]))
        assert abs(got_mean - want_mean) <= 1e-5 * (abs(want_mean) + 1.0)


@pytest.mark.parametrize("K,with_mask,by_source", [(5, True, True), (3, False, False), (1, False, True)])
def test_relational_input_gradient_over_the_batch_view(orc, K, with_mask, by_source):
    """bwd_typed_batch_view: the relational layer's input gradient with rows and edge slots walked in
    ascending order.  Pinned by the dense closed form in fp64 and, where the relation is a function of the
    edge's ends (parallel edges then share it), bit for bit by the weighted backward over the regrouped
    block (orc.typed_csr + orc.bwd_edge_value), which is the per-layer path's order."""
    from helpers import random_csr
    rng = np.random.default_rng(90 + K)
    R, N, F = 70, 40, 6
    ptr, idx = random_csr(rng, R + 20, N, 30, hub=90)
    idx = idx.copy()
    idx[rng.random(len(idx)) < 0.03] = N + 2                    # sources outside the range are dropped
    if by_source:
        rel = (idx * 7 + 3) % (K + 1) - (1 if K > 1 else 0)      # -1 and, for K > 1, every value below K
    else:
        rel = rng.integers(-1, K + 1, size=len(idx))
    rel = rel[: int(ptr[R]) - 4]                                # the last edges have no relation entry
    used = (rng.random(N) < 0.7) if with_mask else None
    g = rng.standard_normal((R * K, F)).astype(np.float32)
    got = orc.bwd_typed_batch_view(ptr, idx, rel, K, g, N, used)
    # closed form
    want = np.zeros((N, F))
    deg = np.diff(ptr)
    for r in range(R):
        for e in range(ptr[r], min(ptr[r + 1], len(rel))):
            s, k = idx[e], rel[e]
            if 0 <= k < K and 0 <= s < N and (used is None or used[s]):
                want[s] += g[r * K + k].astype(np.float64) / deg[r]
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    if used is not None:
        assert (got[~used] == 0).all()
    if by_source:
        ptr2, idx2, cnt, d = orc.typed_csr(ptr, idx, rel, K, R, N, used)
        w2 = orc.typed_csr_weights(ptr2, d, K)
        ref, _, _ = orc.bwd_edge_value(ptr2, idx2, w2, g, None, None, N)
        np.testing.assert_array_equal(got, ref)


def test_edge_types_by_ranges_brute_force(orc):
    from helpers import random_csr
    rng = np.random.default_rng(71)
    R, n_all = 40, 60
    ptr, idx = random_csr(rng, R + 5, n_all, 9)
    s2f = rng.permutation(1000)[:n_all]
    bounds = np.array([300, 650])
    table = np.array([[0, 1, -1], [2, -1, 3], [-1, 4, -1]])
    got = orc.edge_types_by_ranges(ptr, idx, s2f, R, bounds, table)
    typ = lambda v: int(v >= 300) + int(v >= 650)
    for r in range(R + 5):
        for e in range(ptr[r], ptr[r + 1]):
            want = table[typ(s2f[r]), typ(s2f[idx[e]])] if r < R else -1
            assert got[e] == want


def test_evict_by_both_brute_force():
    """Gradient rule then staleness rule against a dictionary model of the table."""
    from oracle import host_model
    rng = np.random.default_rng(77)
    cap, N, M = 60, 200, 40
    for trial in range(5):
        owners = rng.choice(N, size=45, replace=False)
        slots = rng.choice(cap, size=45, replace=False)
        h2f = np.full(cap, -1, np.int64); f2h = np.full(N, -1, np.int64); chk = np.full(cap, -1, np.int64)
        h2f[slots] = owners; f2h[owners] = slots; chk[slots] = rng.integers(0, 12, size=45)
        batch_nodes = rng.choice(N, size=M, replace=False)
        s2h = f2h[batch_nodes].copy()
        s2h[:5] = -1                                              # seeds never use history
        score = rng.random(M).astype(np.float32)
        model = {int(s): (int(o), int(c)) for s, o, c in zip(slots, owners, chk[slots])}
        t = [torch.from_numpy(a) for a in (chk, h2f, f2h, s2h, score)]
        thres = host_model.evict_by_both(t[0], t[1], t[2], t[3], t[4], rate=0.3, glb_iter=12, staleness_thres=6)
        thr = float(thres)
        for r in range(M):
            if s2h[r] != -1 and score[r] >= thr:
                model.pop(int(s2h[r]), None)
        for s in [s for s, (o, c) in model.items() if -1 < c <= 6]:
            model.pop(s)
        want_h2f = np.full(cap, -1, np.int64); want_f2h = np.full(N, -1, np.int64); want_chk = np.full(cap, -1, np.int64)
        for s, (o, c) in model.items():
            want_h2f[s] = o; want_f2h[o] = s; want_chk[s] = c
        np.testing.assert_array_equal(t[1].numpy(), want_h2f)
        np.testing.assert_array_equal(t[2].numpy(), want_f2h)
        np.testing.assert_array_equal(t[0].numpy(), want_chk)
        assert 0 < len(model) < 45


def test_cpu_iteration_of_the_plumbing_configuration(orc):
    """oracle/torch_cpu_path.sage_iteration (the CPU side of `bench.py --workload c1`): the ring it maintains
    stays consistent over iterations that wrap it, admitted rows hold the layer's output, and its admission of
    cached rows are never admitted again."""
    import copy
    from types import SimpleNamespace

    from helpers import layered_batch
    from hiscache import HistorySAGE, make_config       # the model classes need torch only; no GPU is touched
    from oracle import torch_cpu_path as tp
    rng = np.random.default_rng(3)
    torch.manual_seed(3)
    N, Fin, H, C, L = 600, 16, 16, 4, 2                 # in a 2-layer model the cached rows have the input width
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    table = SimpleNamespace(method="grad")
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device="cpu"), table)
    model.table = None
    model = copy.deepcopy(model).train()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2)
    cap = 150                                            # small ring: it wraps
    ring = tp.ring_state(N, cap, H)
    losses = []
    for it in range(1, 9):
        b = layered_batch(rng, N, 30, [5, 4])
        b["y"] = torch.from_numpy(rng.integers(0, C, size=30))
        n1 = int(b["num_node_in_layer"][1])
        before = {k: (v.clone() if torch.is_tensor(v) else v) for k, v in ring.items()}
        losses.append(tp.sage_iteration(model, opt, b, feats, ring, it, 0.5))
        # every mapped node points at a slot that points back; slots written now carry this iteration
        live = torch.nonzero(ring["f2s"] != -1).view(-1)
        assert torch.equal(ring["s2f"][ring["f2s"][live]], live)
        new = torch.nonzero(ring["checkin"] == it).view(-1)
        assert new.numel() > 0 and (ring["header"] - before["header"]) % cap == new.numel() % cap
        ids1 = torch.from_numpy(b["sub_to_full"][:n1])
        assert bool(torch.isin(ring["s2f"][new], ids1).all())
        assert not bool((before["f2s"][ring["s2f"][new]] != -1).any())     # cached rows are not admitted again
    assert all(np.isfinite(losses))
    assert int((ring["checkin"] != -1).sum()) == cap                       # the ring filled up and wrapped
