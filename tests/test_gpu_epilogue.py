"""The hidden layers' epilogue, relu(batch_norm(x + bias)) in training mode, through the C ABI
against torch's own operators in fp64 on the CPU (the reference spells it with
torch.nn.BatchNorm1d and F.relu, /root/reference/hiscache/history_model.py:139-140).
Floating point: 1e-5 relative to each tensor's scale, the bound stated for fp32 paths."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL = 1e-5


def torch_statement(x, bias, gamma, beta, rm, rv, momentum, eps, dy):
    """fp64 on the CPU, operator by operator."""
    x = x.double().cpu().requires_grad_(True)
    bias = None if bias is None else bias.double().cpu().requires_grad_(True)
    gamma = None if gamma is None else gamma.double().cpu().requires_grad_(True)
    beta = None if beta is None else beta.double().cpu().requires_grad_(True)
    rm, rv = rm.double().cpu().clone(), rv.double().cpu().clone()
    z = x if bias is None else x + bias
    y = F.relu(F.batch_norm(z, rm, rv, gamma, beta, True, momentum, eps))
    y.backward(dy.double().cpu())
    g = lambda t: None if t is None else t.grad
    return y.detach(), rm, rv, x.grad, g(bias), g(gamma), g(beta)


def close(got, want, what, rtol=RTOL):
    got, want = got.detach().double().cpu(), want.detach().double()
    scale = float(want.abs().max()) or 1.0
    err = float((got.detach() - want).abs().max())
    assert err <= rtol * scale, f"{what}: max error {err:.3e} against scale {scale:.3e}"


@pytest.mark.parametrize("n,C,offset,affine,with_bias", [
    (2, 4, 0.0, True, True), (37, 8, 5.0, True, False), (1000, 172, 0.0, True, True),
    (5_800, 256, 3.0, True, True), (25_801, 256, 100.0, True, True), (4_162, 1024, 0.0, False, True),
    (70_000, 128, -20.0, True, False), (513, 64, 50.0, True, True)])
def test_bn_relu_matches_torch(n, C, offset, affine, with_bias):
    import hiscache_backend as be
    g = torch.Generator(device=DEV).manual_seed(n * 31 + C)
    rnd = lambda *s: torch.randn(*s, device=DEV, generator=g)
    x = (rnd(n, C) * (1.0 + rnd(C).abs()) + offset + rnd(C)).requires_grad_(True)
    bias = rnd(C).requires_grad_(True) if with_bias else None
    gamma = (1.0 + 0.3 * rnd(C)).requires_grad_(True) if affine else None
    beta = (0.5 * rnd(C)).requires_grad_(True) if affine else None
    rm, rv = rnd(C), rnd(C).abs() + 0.5
    dy = rnd(n, C)
    momentum, eps = 0.1, 1e-5
    # ReLU's derivative jumps at 0: where the fp64 pre-activation is within rounding of 0 the fp32 path may
    # land on the other side, so those elements get no upstream gradient (their y is compared like all others)
    with torch.no_grad():
        z64 = x.double() if bias is None else x.double() + bias.double()
        pre = F.batch_norm(z64, None, None, None if gamma is None else gamma.double(),
                           None if beta is None else beta.double(), True, 0.0, eps)
        ambiguous = pre.abs() < 1e-4 * float(pre.abs().max())
        dy[ambiguous] = 0.0
    want = torch_statement(x.detach(), None if bias is None else bias.detach(),
                           None if gamma is None else gamma.detach(), None if beta is None else beta.detach(),
                           rm, rv, momentum, eps, dy)
    rm1, rv1 = rm.clone(), rv.clone()
    y = be.bias_bn_relu(x, bias, gamma, beta, rm1, rv1, momentum, eps)
    y.backward(dy)
    close(y, want[0], "y")
    # the same elements are clamped, up to the ambiguous ones
    flips = ((y.detach() > 0) != (want[0].to(DEV) > 0)) & ~ambiguous
    assert int(flips.sum()) == 0
    close(rm1, want[1], "running_mean")
    close(rv1, want[2], "running_var")
    # dx is a difference of terms of size |dy| * gamma * invstd (it all but vanishes for n = 2): the bound is
    # relative to those terms
    invstd = 1.0 / torch.sqrt(x.detach().double().var(0, unbiased=False) + eps)
    gscale = float(dy.abs().max()) * float((invstd * (gamma.detach().double().abs() if affine else 1.0)).max())
    assert float((x.grad.double().cpu() - want[3]).abs().max()) <= 2e-5 * gscale
    if with_bias:
        # analytically zero; torch's own value is rounding noise of the same size
        assert float(bias.grad.abs().max()) == 0.0
        assert float(want[4].abs().max()) <= 1e-6 * max(1.0, float(dy.abs().sum(0).max()))
    if affine:
        # the mean is kept in fp32: half an ulp of it shifts every xhat of a column the same way, which dgamma
        # sees multiplied by the column's sum of dy
        mean_ulp = 1.2e-7 * (abs(offset) + 4.0)
        slack = mean_ulp * float(invstd.max()) * float(want[6].abs().max())
        got, ref = gamma.grad.double().cpu(), want[5]
        assert float((got - ref).abs().max()) <= 2e-5 * float(ref.abs().max()) + slack
        close(beta.grad, want[6], "dbeta", 2e-5)
    # same bits on a second call, and the block counter is back at zero
    x2 = x.detach().clone().requires_grad_(True)
    y2 = be.bias_bn_relu(x2, None if bias is None else bias.detach(), None if gamma is None else gamma.detach(),
                         None if beta is None else beta.detach(), rm.clone(), rv.clone(), momentum, eps)
    y2.backward(dy)
    assert torch.equal(y2, y) and torch.equal(x2.grad, x.grad)
    torch.cuda.synchronize()
    assert int(be._ticket(x.device).abs().sum()) == 0


def test_bn_relu_argument_errors():
    import hiscache_backend as be
    x = torch.randn(8, 6, device=DEV)
    with pytest.raises(ValueError):
        be.bias_bn_relu(x, None, None, None, None, None, 0.1, 1e-5)              # C % 4 != 0
    with pytest.raises(ValueError):
        be.bias_bn_relu(torch.randn(1, 8, device=DEV), None, None, None, None, None, 0.1, 1e-5)
    with pytest.raises(ValueError):
        be.bias_bn_relu(torch.randn(8, 8, device=DEV), torch.randn(4, device=DEV), None, None, None, None, 0.1,
                        1e-5)
    with pytest.raises(RuntimeError):
        be.bias_bn_relu(torch.randn(8, 8), None, None, None, None, None, 0.1, 1e-5)


def test_module_bookkeeping_follows_batchnorm1d():
    """Running statistics, batch counter and the cumulative-average mode, over several calls."""
    from hiscache.history_model import bn_relu
    torch.manual_seed(5)
    for momentum in (0.1, None):
        a = torch.nn.BatchNorm1d(64, momentum=momentum).to(DEV).train()
        b = torch.nn.BatchNorm1d(64, momentum=momentum).to(DEV).train()
        b.load_state_dict(a.state_dict())
        bias = torch.randn(64, device=DEV)
        for it in range(4):
            x = torch.randn(300 + it, 64, device=DEV) * 2 + 1
            want = F.relu(a(x + bias))
            got = bn_relu(x, b, bias)
            close(got, want.double().cpu(), "y")
        assert int(a.num_batches_tracked) == int(b.num_batches_tracked) == 4
        close(b.running_mean, a.running_mean.double().cpu(), "running_mean")
        close(b.running_var, a.running_var.double().cpu(), "running_var")
    # evaluation mode and unsupported widths take the torch operators
    a.eval()
    x = torch.randn(10, 64, device=DEV)
    assert torch.equal(bn_relu(x, a, bias), F.relu(a(x + bias)))
    c = torch.nn.BatchNorm1d(6).to(DEV).train()
    x = torch.randn(10, 6, device=DEV)
    c2 = torch.nn.BatchNorm1d(6).to(DEV).train()
    assert torch.allclose(bn_relu(x, c, None), F.relu(c2(x)))


def test_sage_with_fused_epilogue_equals_the_operator_spelling():
    from hiscache import HistorySAGE, PinnedFeatureStore, RingHistoryCache, make_config
    from hiscache.synthetic import make_batch, direct_power_law_batch
    N, Fin, H, C, L = 50_000, 64, 128, 16, 3
    rng = np.random.default_rng(11)
    feats = torch.from_numpy(rng.standard_normal((N, Fin), dtype=np.float32))
    labels = rng.integers(0, C, size=N)
    smp = direct_power_law_batch(N, 200, [5, 4, 3], 2.0, 7, degree_scale=2.0)
    out = {}
    for fused in (True, False):
        torch.manual_seed(2)
        cache = RingHistoryCache(PinnedFeatureStore(feats, device=DEV), N, Fin, H, capacity=N, num_layers=L,
                                 table_dtype=torch.float32, rate=0.5, device=DEV)
        cache.preload(torch.arange(0, N, 3, device=DEV))
        cache.table.normal_(0.0, 0.5, generator=torch.Generator(device=DEV).manual_seed(1))
        model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device=DEV), cache).to(DEV)
        model.fused_epilogue = fused
        model.train()
        b = make_batch(smp, labels, DEV)
        cache.lookup_and_load(b, L)
        logits = model(b)
        F.nll_loss(logits, b.y).backward()
        out[fused] = dict(logits=logits.detach(), his=cache.produced_embedding.grad.clone(),
                          grads={k: p.grad.clone() for k, p in model.named_parameters()},
                          stats={k: v.clone() for k, v in model.state_dict().items() if "running" in k or "num_b" in k})
    close(out[True]["logits"], out[False]["logits"].double().cpu(), "logits", 1e-4)
    close(out[True]["his"], out[False]["his"].double().cpu(), "gradient of the history layer's output", 1e-3)
    for k, v in out[False]["grads"].items():
        if k.endswith("lin_l.bias") and not k.startswith("convs.%d." % (L - 1)):
            # in front of a normalisation: zero here, rounding noise in the operator spelling
            assert float(out[True]["grads"][k].abs().max()) == 0.0
            continue
        close(out[True]["grads"][k], v.double().cpu(), k, 1e-3)
    for k, v in out[False]["stats"].items():
        close(out[True]["stats"][k], v.double().cpu(), k, 1e-5)


@pytest.mark.parametrize("n,H,F,two", [(1, 64, 64, False), (2, 64, 64, True), (63, 128, 64, True), (1000, 192, 128, False),
                                       (5_801, 256, 256, True), (25_817, 256, 128, True), (70_001, 256, 256, True),
                                       (4_096, 512, 320, False), (301, 4096, 4096, False), (129, 64, 4096, True)])
def test_weight_grad_matches_fp64_product(n, H, F, two):
    """hc_weight_grad (matrix cores, slabs added in order) against g^T x in fp64; same bits on a second call."""
    import hiscache_backend as be
    gen = torch.Generator(device=DEV).manual_seed(n + H)
    g = torch.randn(n, H, device=DEV, generator=gen)
    x0 = torch.randn(n + 5, F, device=DEV, generator=gen)[:n]              # a row prefix, as the root rows are
    x1 = torch.randn(n, F, device=DEV, generator=gen) if two else None
    got = be.weight_grad(g, x0, x1)
    got = got if two else (got,)
    for d, x in zip(got, (x0, x1)):
        want = g.double().t() @ x.double()
        scale = float(want.abs().max())
        assert tuple(d.shape) == (H, F)
        assert float((d.double() - want).abs().max()) <= 1e-5 * scale + 1e-6 * (n ** 0.5)
    again = be.weight_grad(g, x0, x1)
    again = again if two else (again,)
    assert all(torch.equal(a, b) for a, b in zip(got, again))
    with pytest.raises(ValueError):
        be.weight_grad(g, torch.randn(n, 48, device=DEV))                 # width off a multiple of 64
    with pytest.raises(ValueError):
        be.weight_grad(g, torch.randn(n, 4160, device=DEV))               # wider than the kernel's limit
    with pytest.raises(ValueError):
        be.weight_grad(g, torch.randn(n + 1, F, device=DEV))              # row counts differ


def test_history_buffer_that_requires_grad_takes_the_operator_spelling():
    """A cached-embedding buffer that asks for a gradient makes the history layer run operator by operator
    (the fused node does not differentiate the buffer); the epilogue still takes the bias and the buffer's
    gradient is the output gradient on the rows that were served from it."""
    from hiscache import HistorySAGE, PinnedFeatureStore, RingHistoryCache, make_config
    from hiscache.synthetic import make_batch, direct_power_law_batch
    N, Fin, H, C, L = 20_000, 64, 64, 8, 3
    rng = np.random.default_rng(5)
    feats = torch.from_numpy(rng.standard_normal((N, Fin), dtype=np.float32))
    smp = direct_power_law_batch(N, 100, [5, 4, 3], 2.0, 9, degree_scale=2.0)
    torch.manual_seed(6)
    cache = RingHistoryCache(PinnedFeatureStore(feats, device=DEV), N, Fin, H, capacity=N, num_layers=L,
                             table_dtype=torch.float32, rate=0.5, device=DEV)
    cache.preload(torch.arange(0, N, 2, device=DEV))
    cache.table.normal_(0.0, 0.5)
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device=DEV), cache).to(DEV).train()
    b = make_batch(smp, rng.integers(0, C, size=N), DEV)
    cache.lookup_and_load(b, L)
    cache.cached_embedding.requires_grad_(True)
    F.nll_loss(model(b), b.y).backward()
    hit = cache.sub2embed != -1
    assert hit.any() and (~hit).any()
    gh = cache.cached_embedding.grad
    assert gh is not None and float(gh[~hit].abs().max()) == 0.0 and float(gh[hit].abs().max()) > 0.0
    pe = cache.produced_embedding
    assert torch.equal(gh[hit], pe.grad[hit])
    assert all(p.grad is not None for p in model.parameters())
