"""The microbenchmark configurations at their full sizes, checked through properties that do not need a
CPU pass over 20 M edges: closed forms on a random sample of rows, weighted column sums (a checksum of
the whole output), the adjoint identity between forward and backward, sortedness and permutation
checksums of the transposed view, the prefix-sum slot rule of the admission pass, and run-to-run
bit-identity.  Reference values are computed with torch ops in fp64 on the device, a path that
shares nothing with the library.  Tolerance: 1e-5 relative for fp32 sums; integer results exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
R, E, N, F = 1_000_000, 20_000_000, 10_000_000, 256


@pytest.fixture(scope="module")
def c2():
    import hiscache_backend as be
    from hiscache.synthetic import power_law_block
    ptr, idx = power_law_block(R, E, N, alpha=2.1, max_degree=5000, seed=2)
    ptr, idx = ptr.to(DEV), idx.to(DEV)
    gen = torch.Generator(device=DEV).manual_seed(2)
    feat = torch.randn(N, F, device=DEV, generator=gen)
    g = torch.randn(R, F, device=DEV, generator=gen)
    hist = 0.5 * torch.randn(N, F, device=DEV, generator=gen)
    hmap = torch.where(torch.rand(N, device=DEV, generator=gen) < 0.4, torch.arange(N, device=DEV),
                       torch.full((N,), -1, device=DEV))
    print("full-size c2 block built", flush=True)
    out = be._aggr_fwd(be.SUBST_SRC, ptr, idx, feat, hmap, hist, F, None, R)
    tr = be.build_transpose(ptr, idx, None, R, N, want_edges=False)
    grad_x, _, _ = be._aggr_bwd(ptr, idx, tr, g, None, None, feat, False, None, 0, R, N)
    torch.cuda.synchronize()
    yield dict(ptr=ptr, idx=idx, feat=feat, g=g, hist=hist, hmap=hmap, out=out, tr=tr, grad_x=grad_x)
    torch.cuda.empty_cache()


def substituted_rows(c, ids):
    """fp64 rows the per-source rule reads for source ids ``ids``."""
    slot = c["hmap"][ids]
    hit = slot != -1
    rows = c["feat"][ids].double()
    rows[hit] = c["hist"][slot[hit]].double()
    return rows


def test_c2_forward_sample_rows_closed_form(c2):
    gen = torch.Generator(device=DEV).manual_seed(11)
    deg = c2["ptr"][1:] - c2["ptr"][:-1]
    sample = torch.randint(0, R, (3000,), device=DEV, generator=gen)
    sample = torch.cat([sample, torch.topk(deg, 8).indices])         # and the longest rows (quarter split)
    starts, ends = c2["ptr"][sample], c2["ptr"][sample + 1]
    worst = 0.0
    for r, b, e in zip(sample.tolist(), starts.tolist(), ends.tolist()):
        want = substituted_rows(c2, c2["idx"][b:e]).sum(0) / max(e - b, 1)
        got = c2["out"][r].double()
        err = float((got - want).abs().max() / want.abs().max().clamp(min=1e-30))
        worst = max(worst, err)
    assert worst < 1e-5, worst


def test_c2_forward_weighted_column_sums(c2):
    """sum_r deg(r) * out[r, :] == sum over all edges of the substituted source row."""
    deg = (c2["ptr"][1:] - c2["ptr"][:-1]).double()
    lhs = (c2["out"].double() * deg[:, None]).sum(0)
    rhs = torch.zeros(F, dtype=torch.float64, device=DEV)
    for lo in range(0, E, 2_000_000):
        rhs += substituted_rows(c2, c2["idx"][lo:lo + 2_000_000]).sum(0)
    scale = float(rhs.abs().max())
    assert float((lhs - rhs).abs().max()) < 1e-5 * scale + 1e-3


def test_c2_adjoint_identity(c2):
    """<fwd(x), g> == <x, bwd(g)> over the substituted source rows (the forward is linear in them)."""
    lhs = float((c2["out"].double() * c2["g"].double()).sum())
    rhs = 0.0
    for lo in range(0, N, 1_000_000):
        ids = torch.arange(lo, min(N, lo + 1_000_000), device=DEV)
        rhs += float((substituted_rows(c2, ids) * c2["grad_x"][ids].double()).sum())
    assert abs(lhs - rhs) < 1e-5 * max(abs(lhs), abs(rhs)) + 1e-2, (lhs, rhs)


def test_c2_backward_sample_sources_closed_form(c2):
    ptrT, rowT, _ = c2["tr"]
    gen = torch.Generator(device=DEV).manual_seed(12)
    deg = (c2["ptr"][1:] - c2["ptr"][:-1]).double()
    sample = torch.randint(0, N, (3000,), device=DEV, generator=gen)
    worst = 0.0
    for s, b, e in zip(sample.tolist(), ptrT[sample].tolist(), ptrT[sample + 1].tolist()):
        rows = rowT[b:e].long()
        want = (c2["g"][rows].double() / deg[rows][:, None]).sum(0)
        got = c2["grad_x"][s].double()
        worst = max(worst, float((got - want).abs().max() / want.abs().max().clamp(min=1e-30)) if e > b
                    else float(got.abs().max()))
    assert worst < 1e-5, worst


def test_c2_transposed_view_is_a_sorted_stable_permutation(c2):
    ptrT, rowT, _ = c2["tr"]
    ptr, idx = c2["ptr"], c2["idx"]
    assert int(ptrT[0]) == 0 and int(ptrT[N]) == E
    seg = ptrT[1:] - ptrT[:-1]
    assert int(seg.min()) >= 0
    # segment sizes are the in-degrees
    assert torch.equal(seg, torch.bincount(idx, minlength=N))
    # inside a segment destination rows ascend (stable sort of a row-major edge list)
    src_of = torch.repeat_interleave(torch.arange(N, device=DEV), seg)
    same = src_of[1:] == src_of[:-1]
    assert bool((rowT[1:][same] >= rowT[:-1][same]).all())
    # the view is a permutation of the edge list: two independent checksums over (source, row) pairs
    row_of = torch.repeat_interleave(torch.arange(R, device=DEV), ptr[1:] - ptr[:-1])
    for a, b in ((1_000_003, 998_244_353), (7, 1_000_000_007)):
        want = int(((idx * a + row_of * b) % 2_147_483_647).sum())
        got = int(((src_of * a + rowT.long() * b) % 2_147_483_647).sum())
        assert want == got


def test_c2_results_are_bit_identical_run_to_run(c2):
    import hiscache_backend as be
    out = be._aggr_fwd(be.SUBST_SRC, c2["ptr"], c2["idx"], c2["feat"], c2["hmap"], c2["hist"], F, None, R)
    assert torch.equal(out, c2["out"])
    tr = be.build_transpose(c2["ptr"], c2["idx"], None, R, N, want_edges=False)
    assert torch.equal(tr[0], c2["tr"][0]) and torch.equal(tr[1], c2["tr"][1])
    grad_x, _, _ = be._aggr_bwd(c2["ptr"], c2["idx"], tr, c2["g"], None, None, c2["feat"], False, None, 0, R, N)
    assert torch.equal(grad_x, c2["grad_x"])


def test_c2_backward_over_the_whole_block_view_has_the_same_bits(c2):
    """hc_aggr_bwd_batch_view at full size: the unfiltered view of the block serves the whole block and
    its first half of the rows (edges of the other rows stepped over in the kernel) with the bits of the
    path that builds a view per call (no source of this block has more than a chunk of incoming edges)."""
    import hiscache_backend as be
    ptrT, rowT, _ = c2["tr"]
    assert int((ptrT[1:] - ptrT[:-1]).max()) <= be.bwd_chunk_edges(F)
    view = be.BatchView(ptrT, rowT, None, R, N, E)
    gx, _ = be._aggr_bwd_batch_view(c2["ptr"], view, c2["g"], None, None, 0, R, N, want_hist_grad=False)
    assert torch.equal(gx, c2["grad_x"])
    del gx
    half = R // 2
    e_half = int(c2["ptr"][half])
    tr_h = be.build_transpose(c2["ptr"], c2["idx"], None, half, N, num_edge=e_half, want_edges=False)
    want, _, _ = be._aggr_bwd(c2["ptr"], c2["idx"], tr_h, c2["g"][:half], None, None, c2["feat"], False, None, 0,
                              half, N)
    got, _ = be._aggr_bwd_batch_view(c2["ptr"], view, c2["g"][:half], None, None, 0, half, N, want_hist_grad=False)
    assert torch.equal(got, want)


def test_c2_every_row_has_the_bits_of_the_cpu_statement(c2):
    """All 1 M output rows, the whole transposed view and all 10 M gradient rows of the full-size block against
    the OpenMP CPU statement (which tests/test_oracle_aggr.py holds to the sequential oracle's bits at small
    sizes): bit for bit.  About 35 GB of host memory at the peak."""
    import hiscache_backend as be
    from oracle import hc_cpu_mt as mt
    ptr, idx = c2["ptr"].cpu().numpy(), c2["idx"].cpu().numpy()
    feat, hist, hmap = c2["feat"].cpu().numpy(), c2["hist"].cpu().numpy(), c2["hmap"].cpu().numpy()
    print("c2 block on the host,", mt.num_threads(), "threads", flush=True)
    want = mt.fwd_mean_src(ptr, idx, feat, hmap, hist, split_above=be.long_row_edges(F))
    got = c2["out"].cpu().numpy()
    bad = int((got.view(np.uint32) != want.view(np.uint32)).any(axis=1).sum())
    assert bad == 0, f"{bad} forward rows differ"
    del feat, hist, want, got
    ptrT, rowT = mt.build_transpose(ptr, idx, N)
    assert np.array_equal(c2["tr"][0].cpu().numpy(), ptrT)
    assert np.array_equal(c2["tr"][1].cpu().numpy()[:E], rowT[:E])
    print("c2 view equal", flush=True)
    want = mt.bwd_mean(ptr, ptrT, rowT, c2["g"].cpu().numpy(), N, chunk=be.bwd_chunk_edges(F))
    got = c2["grad_x"].cpu().numpy()
    bad = int((got.view(np.uint32) != want.view(np.uint32)).any(axis=1).sum())
    assert bad == 0, f"{bad} gradient rows differ"


def test_c4_admission_full_size():
    """2 M rows x 256, fp16 table 50 M x 256: mask == predicate on the kernel's own scores, slots ==
    header + exclusive prefix sum of the mask, table rows == fp16(embedding), maps consistent."""
    import hiscache_backend as be
    from hiscache.synthetic import lognormal_grads
    M, cap = 2_000_000, 50_000_000
    gen = torch.Generator(device=DEV).manual_seed(4)
    grad = lognormal_grads(M, F, -3.0, 1.5, device=DEV, generator=gen)
    emb = torch.randn(M, F, device=DEV, generator=gen)
    age = torch.randint(0, 21, (M,), device=DEV, generator=gen, dtype=torch.int32)
    Nfull = cap
    sub_to_full = torch.randperm(Nfull, device=DEV, generator=gen)[:M].contiguous()
    cached = torch.rand(M, device=DEV, generator=gen) < 0.35
    slot0 = torch.where(cached, torch.randperm(cap, device=DEV, generator=gen)[:M], torch.full((M,), -1, device=DEV))
    table = torch.zeros(cap, F, dtype=torch.float16, device=DEV)
    full2slot = torch.full((Nfull,), -1, dtype=torch.int64, device=DEV)
    slot2full = torch.full((cap,), -1, dtype=torch.int64, device=DEV)
    checkin = torch.full((cap,), -1, dtype=torch.int64, device=DEV)
    header = torch.full((1,), cap - 300_000, dtype=torch.int64, device=DEV)     # the ring wraps inside the call
    thres = torch.tensor([0.05], device=DEV)
    print("full-size c4 block built", flush=True)
    mask, score, slot_out = be.grad_check(grad, emb, slot0, sub_to_full, thres, table, full2slot, slot2full, header,
                                          7, age=age, age_limit=10, checkin=checkin, want_slots=True)
    # scores: the library's summation order against an fp64 norm
    ref = grad.double().norm(dim=1)
    assert float(((score.double() - ref).abs() / ref).max()) < 1e-6
    band = ((score.view(torch.int32) - thres.view(torch.int32)).abs() <= 4).sum()
    print("rows within 4 ulp of the threshold:", int(band), flush=True)
    want = (score < thres) & ((slot0 == -1) | (age >= 10))
    assert torch.equal(mask, want)
    A = int(mask.sum())
    assert 700_000 < A < 950_000
    # all 2 M scores have the bits of the CPU statement's summation order (portable build: separately rounded
    # multiplies and adds, which tests/test_oracle_admission.py holds to the sequential oracle)
    from oracle import hc_cpu_mt as mt
    cpu_score = mt.score_rows(grad.cpu().numpy(), hw=False)
    assert np.array_equal(score.cpu().numpy().view(np.uint32), cpu_score.view(np.uint32))
    rank = torch.cumsum(mask.long(), 0) - mask.long()
    want_slot = torch.where(mask, (cap - 300_000 + rank) % cap, torch.full_like(rank, -1))
    assert torch.equal(slot_out, want_slot)
    assert int(header) == (cap - 300_000 + A) % cap
    s = slot_out[mask]
    assert torch.equal(table[s], emb[mask].half())
    assert torch.equal(slot2full[s], sub_to_full[mask]) and torch.equal(full2slot[sub_to_full[mask]], s)
    assert bool((checkin[s] == 7).all()) and int((checkin != -1).sum()) == A
    assert int((slot2full != -1).sum()) == A and int((full2slot != -1).sum()) == A
    # a second identical call admits the same rows into the next slots and un-maps nothing it should not
    mask2, _, slot2 = be.grad_check(grad, emb, slot0, sub_to_full, thres, table, full2slot, slot2full, header,
                                    8, age=age, age_limit=10, checkin=checkin, want_slots=True)
    assert torch.equal(mask2, mask)
    assert torch.equal(slot2[mask], (s + A) % cap)
    assert int((full2slot != -1).sum()) == A                 # same nodes, moved to their new slots
    assert torch.equal(full2slot[sub_to_full[mask]], slot2[mask])


def test_c2_view_without_substituted_sources(c2):
    """The view the benchmark's step builds (edges of substituted sources left out) against the full one:
    exactly the edges of unsubstituted sources, in the same order, hence the same bits in their gradient
    rows; substituted sources get empty segments and zero rows."""
    import hiscache_backend as be
    ptrT_f, rowT_f, _ = c2["tr"]
    tr = be.build_transpose(c2["ptr"], c2["idx"], None, R, N, want_edges=False, history_map_src=c2["hmap"])
    ptrT, rowT, _ = tr
    sub = c2["hmap"] != -1
    seg_f, seg = ptrT_f[1:] - ptrT_f[:-1], ptrT[1:] - ptrT[:-1]
    assert int(ptrT[0]) == 0
    assert torch.equal(seg, torch.where(sub, torch.zeros_like(seg_f), seg_f))
    live = int(ptrT[N])
    assert live == int((~sub[c2["idx"]]).sum()) and 0.55 * E < live < 0.65 * E
    keep = torch.repeat_interleave(~sub, seg_f)               # transposed edges of the full view that stay
    assert torch.equal(rowT[:live], rowT_f[keep])
    grad_x, _, _ = be._aggr_bwd(c2["ptr"], c2["idx"], tr, c2["g"], None, None, c2["feat"], False, None, 0, R, N)
    assert float(grad_x[sub].abs().max()) == 0.0
    assert torch.equal(grad_x[~sub], c2["grad_x"][~sub])


# ------------------------------------------------------------------------------------------------
# The papers100M-shaped history layer of about 800 sampled batches side by side (4.7 M rows, 20 M edges,
# 20.8 M sources x 256, 35% of the rows taken from an fp16 row-aligned history buffer): the block whose
# forward + view + backward + admission the benchmark reports as kernels.c3_batched.
@pytest.fixture(scope="module")
def c3b():
    import hiscache_backend as be
    from hiscache.synthetic import batched_history_layer, direct_power_law_batch
    samples = [direct_power_law_batch(111_000_000, 1000, [15, 10, 5], 2.0, 30 + i, degree_scale=2.6) for i in range(8)]
    ptr_h, idx_h, Rb, Eb, Nb = batched_history_layer(samples, 20_000_000)
    ptr, idx = torch.from_numpy(ptr_h).to(DEV), torch.from_numpy(idx_h).to(DEV)
    gen = torch.Generator(device=DEV).manual_seed(33)
    x = torch.randn(Nb, F, device=DEV, generator=gen)
    hbuf = (0.5 * torch.randn(Rb, F, device=DEV, generator=gen)).half()
    hmap = torch.where(torch.rand(Rb, device=DEV, generator=gen) < 0.35, torch.arange(Rb, device=DEV),
                       torch.full((Rb,), -1, device=DEV))
    g = torch.randn(Rb, F, device=DEV, generator=gen)
    print("full-size batched history layer built: %d rows, %d edges, %d sources" % (Rb, Eb, Nb), flush=True)
    out = be._aggr_fwd(be.SUBST_ROW, ptr, idx, x, hmap, hbuf, F, None, Rb)
    tr = be.build_transpose(ptr, idx, hmap, Rb, Nb, want_edges=False)
    grad_x, _, _ = be._aggr_bwd(ptr, idx, tr, g, hmap, None, x, False, (Rb, F), F, Rb, Nb, want_hist_grad=False)
    torch.cuda.synchronize()
    yield dict(ptr=ptr, idx=idx, x=x, hbuf=hbuf, hmap=hmap, g=g, out=out, tr=tr, grad_x=grad_x, R=Rb, E=Eb, N=Nb)
    torch.cuda.empty_cache()


def test_c3_batched_forward(c3b):
    c = c3b
    hit = c["hmap"] != -1
    assert 4_000_000 < c["R"] < 6_000_000 and c["E"] >= 20_000_000 and 0.33 < float(hit.float().mean()) < 0.37
    # history rows carry the fp16 buffer row exactly
    assert torch.equal(c["out"][hit], c["hbuf"][hit].float())
    # computed rows: closed form on a sample, and the degree-weighted column sums of all of them
    gen = torch.Generator(device=DEV).manual_seed(21)
    deg = c["ptr"][1:] - c["ptr"][:-1]
    cand = torch.nonzero(~hit).view(-1)
    sample = cand[torch.randint(0, cand.numel(), (3000,), device=DEV, generator=gen)]
    sample = torch.cat([sample, cand[torch.topk(deg[cand], 8).indices]])
    worst = 0.0
    for r, b, e in zip(sample.tolist(), c["ptr"][sample].tolist(), c["ptr"][sample + 1].tolist()):
        want = c["x"][c["idx"][b:e]].double().sum(0) / max(e - b, 1)
        got = c["out"][r].double()
        worst = max(worst, float((got - want).abs().max() / want.abs().max().clamp(min=1e-30)) if e > b
                    else float(got.abs().max()))
    assert worst < 1e-5, worst
    w = torch.where(hit, torch.zeros_like(deg), deg).double()
    lhs = (c["out"].double() * w[:, None]).sum(0)
    row_of = torch.repeat_interleave(torch.arange(c["R"], device=DEV), deg)
    rhs = torch.zeros(F, dtype=torch.float64, device=DEV)
    for lo in range(0, c["E"], 2_000_000):
        sl = slice(lo, lo + 2_000_000)
        keep = ~hit[row_of[sl]]
        rhs += c["x"][c["idx"][sl][keep]].double().sum(0)
    assert float((lhs - rhs).abs().max()) < 1e-5 * float(rhs.abs().max()) + 1e-3


def test_c3_batched_every_row_has_the_oracles_bits(c3b):
    """All 4.7 M output rows (history rows from the fp16 buffer included) and all 20.8 M gradient rows of the
    batched layer against the sequential CPU oracle, bit for bit.  About 60 GB of host memory at the peak."""
    import hiscache_backend as be
    from oracle import hc_oracle as orc
    c = c3b
    ptr, idx, hmap = c["ptr"].cpu().numpy(), c["idx"].cpu().numpy(), c["hmap"].cpu().numpy()
    x = c["x"].cpu().numpy()
    hbuf = c["hbuf"].float().cpu().numpy()
    print("batched layer on the host", flush=True)
    want = orc.fwd_mean_row(ptr, idx, x, hmap, hbuf, split_above=be.long_row_edges(F))
    got = c["out"].cpu().numpy()
    bad = int((got.view(np.uint32) != want.view(np.uint32)).any(axis=1).sum())
    assert bad == 0, f"{bad} forward rows differ"
    del x, hbuf, want, got
    print("batched layer: forward equal", flush=True)
    want, _ = orc.bwd_mean_row(ptr, idx, c["g"].cpu().numpy(), hmap, c["N"], (c["R"], F),
                               chunk=be.bwd_chunk_edges(F))
    got = c["grad_x"].cpu().numpy()
    bad = int((got.view(np.uint32) != want.view(np.uint32)).any(axis=1).sum())
    assert bad == 0, f"{bad} gradient rows differ"


def test_c3_batched_view_and_backward(c3b):
    c = c3b
    ptrT, rowT, _ = c["tr"]
    hit = c["hmap"] != -1
    deg = c["ptr"][1:] - c["ptr"][:-1]
    row_of = torch.repeat_interleave(torch.arange(c["R"], device=DEV), deg)
    live = ~hit[row_of]
    n_live = int(live.sum())
    assert int(ptrT[0]) == 0 and int(ptrT[c["N"]]) == n_live
    seg = ptrT[1:] - ptrT[:-1]
    assert torch.equal(seg, torch.bincount(c["idx"][live], minlength=c["N"]))
    src_of = torch.repeat_interleave(torch.arange(c["N"], device=DEV), seg)
    same = src_of[1:] == src_of[:-1]
    rt = rowT[:n_live]
    assert bool((rt[1:][same] >= rt[:-1][same]).all())
    assert not bool(hit[rt.long()].any())                      # no edge of a history row survives
    for a, b in ((1_000_003, 998_244_353), (7, 1_000_000_007)):
        want = int(((c["idx"][live] * a + row_of[live] * b) % 2_147_483_647).sum())
        got = int(((src_of * a + rt.long() * b) % 2_147_483_647).sum())
        assert want == got
    # backward: closed form on sampled sources, then the adjoint identity over the computed rows
    gen = torch.Generator(device=DEV).manual_seed(22)
    sample = torch.randint(0, c["N"], (3000,), device=DEV, generator=gen)
    sample = torch.cat([sample, torch.topk(seg, 8).indices])
    degd = deg.double()
    worst = 0.0
    for s_, b, e in zip(sample.tolist(), ptrT[sample].tolist(), ptrT[sample + 1].tolist()):
        rows = rowT[b:e].long()
        got = c["grad_x"][s_].double()
        if e > b:
            want = (c["g"][rows].double() / degd[rows][:, None]).sum(0)
            worst = max(worst, float((got - want).abs().max() / want.abs().max().clamp(min=1e-30)))
        else:
            worst = max(worst, float(got.abs().max()))
    assert worst < 1e-5, worst
    lhs = float((c["out"].double() * c["g"].double())[~hit].sum())
    rhs = 0.0
    for lo in range(0, c["N"], 2_000_000):
        rhs += float((c["x"][lo:lo + 2_000_000].double() * c["grad_x"][lo:lo + 2_000_000].double()).sum())
    assert abs(lhs - rhs) < 1e-5 * max(abs(lhs), abs(rhs)) + 1e-2, (lhs, rhs)


def test_c3_batched_admission_and_bit_identity(c3b):
    import hiscache_backend as be
    from hiscache.synthetic import lognormal_grads
    c = c3b
    Rb = c["R"]
    gen = torch.Generator(device=DEV).manual_seed(34)
    grad = lognormal_grads(Rb, F, -3.0, 1.5, device=DEV, generator=gen)
    cap = max(Rb, 1 << 20)
    table = torch.zeros(cap, F, dtype=torch.float16, device=DEV)
    f2s = torch.full((2 * Rb,), -1, dtype=torch.int64, device=DEV)
    s2f = torch.full((cap,), -1, dtype=torch.int64, device=DEV)
    chk = torch.full((cap,), -1, dtype=torch.int64, device=DEV)
    hdr = torch.zeros(1, dtype=torch.int64, device=DEV)
    sub_to_full = torch.randperm(2 * Rb, device=DEV, generator=gen)[:Rb].contiguous()
    thr = torch.tensor([0.05], device=DEV)
    # the layer's own output is what gets admitted, the rows' slots are the history map
    mask, score, slots = be.grad_check(grad, c["out"], c["hmap"], sub_to_full, thr, table, f2s, s2f, hdr, 1,
                                       checkin=chk, want_slots=True)
    want = (score < thr) & (c["hmap"] == -1)
    assert torch.equal(mask, want)
    A = int(mask.sum())
    assert 0.25 * Rb < A < 0.45 * Rb and int(hdr) == A % cap
    rank = torch.cumsum(mask.long(), 0) - mask.long()
    assert torch.equal(slots, torch.where(mask, rank % cap, torch.full_like(rank, -1)))
    s_ = slots[mask]
    assert torch.equal(table[s_], c["out"][mask].half())
    assert torch.equal(s2f[s_], sub_to_full[mask]) and torch.equal(f2s[sub_to_full[mask]], s_)
    assert int((f2s != -1).sum()) == A and bool((chk[s_] == 1).all())
    # forward, view and backward give the same bits when run again
    out = be._aggr_fwd(be.SUBST_ROW, c["ptr"], c["idx"], c["x"], c["hmap"], c["hbuf"], F, None, Rb)
    assert torch.equal(out, c["out"])
    tr = be.build_transpose(c["ptr"], c["idx"], c["hmap"], Rb, c["N"], want_edges=False)
    n_live = int(tr[0][-1])
    assert torch.equal(tr[0], c["tr"][0]) and torch.equal(tr[1][:n_live], c["tr"][1][:n_live])
    grad_x, _, _ = be._aggr_bwd(c["ptr"], c["idx"], tr, c["g"], c["hmap"], None, c["x"], False, (Rb, F), F, Rb, c["N"],
                                want_hist_grad=False)
    assert torch.equal(grad_x, c["grad_x"])
