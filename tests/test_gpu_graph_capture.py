"""The entry points under HIP graph capture: nothing in them allocates or synchronises, so a caller
may record them.  Every replay is checked against the eager result, with eager work and
synchronisations between the replays and fresh input values for each of them."""
import numpy as np
import pytest
import torch

from helpers import random_csr, random_hmap

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def be():
    import hiscache_backend
    hiscache_backend.load_library()
    return hiscache_backend


def test_aggregation_and_admission_replay_like_eager(be):
    if be.CHECK_INPUTS:
        pytest.skip("HISCACHE_CHECK_INPUTS=1 validates every block with a read-back, which cannot be captured")
    rng = np.random.default_rng(90)
    R, N, F, cap = 3000, 2500, 128, 4096
    ptr, idx = random_csr(rng, R, N, 9, hub=700)
    hmap = random_hmap(rng, R, 0.3)
    T = lambda a: torch.from_numpy(a).to(DEV)
    ptr_d, idx_d, hmap_d = T(ptr), T(idx), T(hmap)
    x = torch.zeros(N, F, device=DEV)
    hbuf = torch.zeros(R, F, device=DEV)
    g = torch.zeros(R, F, device=DEV)
    emb = torch.zeros(R, F, device=DEV)
    slot = torch.full((R,), -1, dtype=torch.int64, device=DEV)
    sub_to_full = T(rng.permutation(3 * R)[:R].astype(np.int64))
    thres = torch.tensor([11.3], device=DEV)          # about the median norm of a 128-dim N(0,1) row
    gather_ids = T(rng.integers(0, N, size=2000).astype(np.int64))
    N_all = max(R, N)
    E = int(ptr[-1])
    sizes = T(np.array([R, E, N], np.int64))          # the block's sizes as the sampler leaves them: on the device
    bn_bias, bn_gamma, bn_beta = (torch.randn(F, device=DEV) for _ in range(3))

    def fresh_state():
        return dict(table=torch.zeros(cap, F, dtype=torch.float16, device=DEV),
                    full2slot=torch.full((3 * R,), -1, dtype=torch.int64, device=DEV),
                    slot2full=torch.full((cap,), -1, dtype=torch.int64, device=DEV),
                    header=torch.zeros(1, dtype=torch.int64, device=DEV),
                    running_mean=torch.zeros(F, device=DEV), running_var=torch.ones(F, device=DEV),
                    batches=torch.zeros((), dtype=torch.int64, device=DEV))

    def work(st):
        out = be._aggr_fwd(be.SUBST_ROW, ptr_d, idx_d, x, hmap_d, hbuf, F, None, R)
        tr = be.build_transpose(ptr_d, idx_d, hmap_d, R, N, want_edges=False)
        gx, gh, _ = be._aggr_bwd(ptr_d, idx_d, tr, g, hmap_d, None, x, False, (R, F), F, R, N)
        mask, score = be.grad_check(g, emb, slot, sub_to_full, thres, st["table"], st["full2slot"], st["slot2full"],
                                    st["header"], 3)
        rows = be.gather_rows(x, gather_ids)             # more rows than the capped grid of a host-memory table
        found = be.lookup(st["full2slot"], sub_to_full, 0)
        used = torch.stack(be.count_history_reconstruct(ptr_d, idx_d, hmap_d[:R], N_all, 64, 2))
        # a hidden layer's epilogue (its block counter is left at zero by every launch) and its backward
        zin = out.detach().requires_grad_(True)
        act = be.bias_bn_relu(zin, bn_bias, bn_gamma, bn_beta, st["running_mean"], st["running_var"], 0.1, 1e-5,
                              st["batches"])
        (dz,) = torch.autograd.grad(act, zin, g)
        # the whole block's view built with the sizes read on the device (capacities above the sizes), and the
        # backward over it with the history rows stepped over in the kernel
        vp, vr, _ = be.build_transpose_dev(ptr_d, idx_d, sizes[0:1], sizes[1:2], sizes[2:3], E, N + 100)
        view = be.BatchView(vp[: N + 1], vr, None, R, N, E)
        gx_v, gh_v = be._aggr_bwd_batch_view(ptr_d, view, g, hmap_d, (R, F), F, R, N)
        return out, tr[0], tr[1], gx, gh, mask, score, rows, found, used, act.detach(), dz, vp[: N + 1], gx_v, gh_v

    def load_inputs(seed):
        gen = torch.Generator(device=DEV).manual_seed(seed)
        for t in (x, hbuf, g, emb):
            t.copy_(torch.randn(t.shape, device=DEV, generator=gen))

    load_inputs(0)
    st_graph = fresh_state()
    work(st_graph)                                   # warm-up outside capture (library handles, allocator pools)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = work(st_graph)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(1, 5):
        load_inputs(rep)
        for k, v in fresh_state().items():
            st_graph[k].copy_(v)
        st_eager = fresh_state()
        eager = work(st_eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("out", "ptrT", "rowT", "grad_x", "grad_h", "mask", "score", "rows", "found", "used",
                               "epilogue", "epilogue gradient", "ptrT of the whole block", "grad_x over it",
                               "grad_h over it"), captured, eager):
            if name == "rowT":                     # only the first ptrT[-1] entries are defined
                n_tr = int(eager[1][-1])
                a, b = a[:n_tr], b[:n_tr]
            assert torch.equal(a, b), (rep, name)
        for k in st_eager:
            assert torch.equal(st_graph[k], st_eager[k]), (rep, k)
        assert 0 < int(st_eager["header"]) < R
        assert int(st_eager["batches"]) == 1
        assert torch.equal(eager[4], eager[14])        # the history rows' gradient does not depend on the view


def test_large_transposed_build_is_captured_and_replayed(be):
    """Above 2^20 edge slots the view comes from the library's own bucket sort, which is kernels only: the
    call is recorded, and every replay (fresh edges between the replays) gives the eager result."""
    R, N, deg = 300_000, 50_000, 4
    E = R * deg
    assert E > 1 << 20
    gen = torch.Generator(device=DEV).manual_seed(7)
    ptr = torch.arange(R + 1, device=DEV, dtype=torch.int64) * deg
    idx = torch.randint(0, N, (E,), device=DEV, generator=gen)
    hsrc = torch.where(torch.rand(N, device=DEV, generator=gen) < 0.3, 1, -1).to(torch.int64)
    be.build_transpose(ptr, idx, None, R, N, want_edges=False, history_map_src=hsrc)   # sizes the workspace pool
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            got = be.build_transpose(ptr, idx, None, R, N, want_edges=False, history_map_src=hsrc)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        idx.copy_(torch.randint(0, N, (E,), device=DEV, generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        eager = be.build_transpose(ptr, idx, None, R, N, want_edges=False, history_map_src=hsrc)
        n_tr = int(eager[0][-1])
        assert torch.equal(got[0], eager[0]), rep
        assert torch.equal(got[1][:n_tr], eager[1][:n_tr]), rep


def test_transposed_build_beyond_the_bucket_sort_is_refused_on_a_capturing_stream(be):
    """More sources than the bucket sort takes (about 44 M) with more than 2^20 edge slots: the sort library
    underneath would record memset nodes, so the call returns an error on a capturing stream, records nothing,
    and works again once the capture is over."""
    R, N, deg = 300_000, 46_000_000, 4
    E = R * deg
    assert E > 1 << 20
    gen = torch.Generator(device=DEV).manual_seed(7)
    ptr = torch.arange(R + 1, device=DEV, dtype=torch.int64) * deg
    idx = torch.randint(0, N, (E,), device=DEV, generator=gen)
    eager = be.build_transpose(ptr, idx, None, R, N, want_edges=False)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(ValueError):
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                kept = idx + 1                          # the capture is not empty
                be.build_transpose(ptr, idx, None, R, N, want_edges=False)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    again = be.build_transpose(ptr, idx, None, R, N, want_edges=False)
    assert torch.equal(again[0], eager[0]) and torch.equal(again[1][:E], eager[1][:E])
