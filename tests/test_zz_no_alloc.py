"""hc_grad_check_static (the admission entry point that allocates nothing: its scratch is a fixed
device array inside the library) against hc_grad_check on the same inputs, bit for bit, on two
calls in a row, the second on a smaller input (so the array still holds what the first call left),
then against the CPU oracle.  Collected last: it must pass alone in a fresh process and after
every other test."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _case(rng, N, M, F, f2s):
    sub_to_full = rng.choice(N, size=M, replace=False).astype(np.int64)
    grad = (rng.standard_normal((M, F)) * np.exp(rng.normal(-3, 1.5, size=(M, 1)))).astype(np.float32)
    emb = rng.standard_normal((M, F)).astype(np.float32)
    age = rng.integers(0, 21, size=M).astype(np.int32)
    used = rng.random(M) < 0.9
    return dict(sub_to_full=sub_to_full, grad=grad, emb=emb, age=age, used=used, slot=f2s[sub_to_full].copy())


def _ring(N, cap, F):
    return dict(table=np.zeros((cap, F), np.uint16), f2s=np.full(N, -1, np.int64), s2f=np.full(cap, -1, np.int64),
                checkin=np.full(cap, -1, np.int64), header=np.array([cap - 77], np.int64))


def _run(be, state, c, it, static):
    return be.grad_check(T(c["grad"]), T(c["emb"]), T(c["slot"]), T(c["sub_to_full"]),
                         torch.tensor([0.05], device=DEV), state["table"], state["f2s"], state["s2f"],
                         state["header"], it, age=T(c["age"]), age_limit=10, used=T(c["used"]),
                         checkin=state["checkin"], want_slots=True, static_scratch=static)


def test_static_scratch_admission_matches_workspace_admission(orc):
    import hiscache_backend as be
    be.load_library()
    rng = np.random.default_rng(77)
    N, cap, F = 200_000, 30_000, 256
    ref = _ring(N, cap, F)
    a = {k: T(v) for k, v in ref.items()}
    b = {k: T(v) for k, v in ref.items()}
    for s in (a, b):
        s["table"] = s["table"].view(torch.float16)
    # second call smaller than the first: 40 000 rows = 625 tiles = 20 chunks, then 5 000 rows = 79 tiles
    for it, M in enumerate([40_000, 5_000, 129]):
        c = _case(rng, N, M, F, ref["f2s"])
        got_s = _run(be, a, c, it, True)
        got_w = _run(be, b, c, it, False)
        torch.cuda.synchronize()
        for x, y, name in zip(got_s, got_w, ("mask", "score", "slots")):
            assert torch.equal(x, y), f"{name} differs at call {it}"
        for k in a:
            assert torch.equal(a[k].view(torch.int16) if k == "table" else a[k],
                               b[k].view(torch.int16) if k == "table" else b[k]), f"{k} differs at call {it}"
        rmask, rscore, rslots = orc.grad_check(c["grad"], c["emb"], c["slot"], c["age"], c["used"], c["sub_to_full"],
                                               0.05, 10, orc.NORM_L2, orc.CMP_LT, ref["table"], orc.DT_F16,
                                               ref["f2s"], ref["s2f"], ref["checkin"], ref["header"], it)
        np.testing.assert_array_equal(got_s[0].cpu().numpy(), rmask)
        np.testing.assert_array_equal(got_s[1].cpu().numpy(), rscore)
        np.testing.assert_array_equal(got_s[2].cpu().numpy(), rslots)
        for k in ("f2s", "s2f", "checkin", "header"):
            np.testing.assert_array_equal(a[k].cpu().numpy(), ref[k], err_msg=f"{k} at call {it}")
        live = ref["s2f"] != -1
        np.testing.assert_array_equal(a["table"].view(torch.int16).cpu().numpy().view(np.uint16)[live],
                                      ref["table"][live])
        assert rmask.sum() > 0


def test_static_scratch_rejects_more_rows_than_it_holds():
    import hiscache_backend as be
    lib = be.load_library()
    M = be.GRAD_CHECK_STATIC_MAX_ROWS + 1
    one = torch.zeros(1, device=DEV)
    h = torch.zeros(1, dtype=torch.int64, device=DEV)
    p = be._ptr
    # the size check comes before any pointer is used: nothing is launched
    rc = lib.hc_grad_check_static(p(one), None, p(one), p(h), None, None, p(h), p(one), 0, 0, 0, p(h), None, None,
                                  p(one), 0, 1, p(h), p(h), None, p(h), 0, M, 256, None)
    assert rc == 5   # HC_EUNSUPPORTED
