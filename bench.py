#!/usr/bin/env python3
"""Benchmark of the HisCache hot path on one MI355X.

Default workload ("c2", the aggregation microbenchmark the metric is quoted on):
  CSR block with 1M destination rows and 20M edges (Zipf alpha=2.1 degrees, max 5000), source ids
  uniform over 10M nodes, 40% of which hit a 10M x 256 fp32 history table (the rest read a
  10M x 256 fp32 feature matrix); mean aggregation forward, then backward with upstream ~N(0,1).
A step = forward + transposed-view build + backward over that block, inputs resident in HBM.

Prints ONE JSON line: edges/s over the whole step, the roofline of the dominant kernel (the forward
gather, timed with HIP events on the launch stream) and a CPU baseline (the same semantics written
with PyTorch CPU index_add, timed on this machine's host cores on a 1/10-size sample).

The default line also carries the admission microbenchmark (c4), the papers100M-shaped history layer
batched to 20 M edges (kernels.c3_batched) and the per-iteration time of the papers100M- and
mag240M-shaped training iterations at their real batch shapes (iterations.c3, iterations.c5), of the
CPU-runnable plumbing configuration beside its PyTorch CPU spelling (iterations.c1) and of the
papers100M-shaped one fed by the device sampler with the features read one batch ahead (iterations.c3_sampled);
--headline-only leaves them out.
Other workloads (--workload c4 | c2row | c3 | c5 ...) print their own line and are not the headline.
"""
import argparse
import gc
import json
import os
import sys
import time
import types

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "history-cache_amd"))

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch at full size, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file (FETCH_SIZE
# scaled by 2.000, WRITE_SIZE by 1.000: factors from a 4 GiB device copy; profiles/aggr_c2_hbm_traffic.md): the
# forward gather of c2 / c2row, the three admission passes of c4, forward + backward + admission of the batched layer.
# Age limit of the ring caches in the iteration workloads: entries preloaded at iteration 0 must stay valid
# for the whole run so that the hit rate stays at the configuration's 35% (the age bound itself is exercised
# by the c4 workload and by the tests).
AGE_LIMIT_ITERS = 100_000
# the c3 / c5 training iterations that the default line reports beside the kernels' figures
ITERATION_STEPS, ITERATION_WARMUP = 200, 20
# HBM bytes per launch by the counters (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 4 GiB copy), measured
# with the library built from commit 6072fbd: profiles/aggr_c2_hbm_traffic.md, rows "C2 fwd_mean_fast" (c2),
# "C4 gc_pass1 + gc_pass3_ring" (c4) and the three "batched layer" rows (c3_batched); c2row from the same
# procedure over `--workload c2row` at commit 173ecbf (that kernel has not changed since).
MEASURED_TRAFFIC = {"c2": 23.08e9, "c2row": 13.93e9, "c4": 3.49e9, "c3_batched": 51.97e9}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--with-sampler", action="store_true",
                    help="c3: draw every batch with the device sampler from a papers100M-sized graph in HBM "
                         "(next batch sampled on a side stream) instead of taking pre-generated batches")
    ap.add_argument("--prefetch", action="store_true",
                    help="c3/c5: start each batch's host-link feature read one batch ahead, on a side stream, for "
                         "the rows that the cache's state at that moment makes necessary (fixed up at the lookup)")
    ap.add_argument("--hot-fraction", type=float, default=0.0,
                    help="c3 --with-sampler: copies of this share of the feature rows, the nodes with the most "
                         "incoming edges, are kept in device memory; only the other rows cross the host link")
    ap.add_argument("--prefetch-cus", type=int, default=16,
                    help="with --prefetch: compute units the read-ahead's stream may use (0: an ordinary stream)")
    ap.add_argument("--prefetch-depth", type=int, default=1,
                    help="with --prefetch and --with-sampler: batches whose feature read is under way")
    ap.add_argument("--prefetch-all", action="store_true",
                    help="with --prefetch: read every row of the next batch and mask at the lookup")
    ap.add_argument("--features-in-hbm", action="store_true",
                    help="c3: the node features live in device memory instead of pinned host memory (a variant beside "
                         "the configuration's own placement: 288 GB hold the papers100M-sized matrix, 57 GB, next to "
                         "the 57 GB history table; the mag240M-sized one, 187 GB beside a 125 GB table, does not fit)")
    ap.add_argument("--sampler-replay", type=int, default=4,
                    help="c1 / c3 --with-sampler: slots of the device sampler whose launches are recorded in HIP graphs "
                         "and replayed, one launch per batch (0: every batch is launched kernel by kernel)")
    ap.add_argument("--recorded", action="store_true",
                    help="c1/c3/c5: the iteration is recorded once per padded batch shape in a HIP graph and replayed "
                         "(hiscache.RecordedIteration) instead of being enqueued operator by operator")
    ap.add_argument("--no-batch-view", action="store_true",
                    help="c3/c5: batches come without the transposed view of their CSR, so every layer's "
                         "backward builds one (the default: the loader emits it with the batch)")
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c2row", "c2w", "c4", "c3", "c3b", "c5", "sample", "layer", "copy", "trainer", "dispatch"])
    ap.add_argument("--heads", type=int, default=1, help="c2w: heads of the weighted aggregation (divides 256)")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the workload (testing only)")
    ap.add_argument("--reps", type=int, default=8, help="c3b: measurements with freshly allocated tensors")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="c2: skip the c4 and batched-c3 kernel figures and the c3 / c5 iteration figures that "
                         "the default run adds to its line")
    return ap.parse_args()


def sync():
    import torch
    torch.cuda.synchronize()


def host_threads():
    """Threads for the CPU baselines: the box's CPU share (OMP_NUM_THREADS where it is set), 16 at most."""
    try:
        n = int(os.environ.get("OMP_NUM_THREADS", "0"))
    except ValueError:
        n = 0
    if n <= 0:
        n = os.cpu_count() or 1
    return max(1, min(n, 16))


def timed_steps(step, steps, warmup):
    """W untimed steps, then exactly K steps between two synchronisations."""
    for _ in range(warmup):
        step()
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    sync()
    return (time.perf_counter() - t0) / steps


class KernelClock:
    """HIP-event timing of one launch site on the current stream, accumulated over the timed region."""

    enabled = True                  # off: the wrapped call runs bare (its events cost the host 5 - 10 us a pair)

    def __init__(self):
        self.pairs = []
        self.cpu_s = 0.0            # host time spent inside fn (enqueueing; nothing here waits for the GPU)

    def __call__(self, fn):
        if not KernelClock.enabled:
            return fn()
        import torch
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        t0 = time.perf_counter()
        out = fn()
        self.cpu_s += time.perf_counter() - t0
        b.record()
        self.pairs.append((a, b))
        return out

    def reset(self):
        self.pairs = []
        self.cpu_s = 0.0

    def mean_cpu_ms(self):
        return 1e3 * self.cpu_s / max(1, len(self.pairs))

    def mean_ms(self):
        return sum(a.elapsed_time(b) for a, b in self.pairs) / max(1, len(self.pairs))


def backward_on_this_thread(loss):
    """``loss.backward()`` without the hand-over to autograd's device thread (``hiscache.backward_on_this_thread``);
    HISCACHE_BENCH_AUTOGRAD_THREAD=1 keeps the hand-over, for comparison."""
    if os.environ.get("HISCACHE_BENCH_AUTOGRAD_THREAD", "0") not in ("", "0"):
        loss.backward()
        return
    from hiscache import backward_on_this_thread as run
    run(loss)


PHASE_STEPS = 100
LAST_CHUNKS = []          # ms per iteration of every chunk (an eighth of the steps) of the last bare pass


def chunk_figures():
    """Median and range of the per-chunk figures of the last ``time_iterations`` pass (device timeline)."""
    c = sorted(LAST_CHUNKS)
    if not c:
        return None
    return {"median": c[len(c) // 2] if len(c) % 2 else 0.5 * (c[len(c) // 2 - 1] + c[len(c) // 2]),
            "min": c[0], "max": c[-1], "chunks": len(c)}


def time_iterations(step, steps, clocks, reset=None):
    """``steps`` iterations timed bare (sync, clock, sync), then up to PHASE_STEPS more with the per-phase event clocks
    switched on for the phase figures: the events of five phases cost a host-bound loop 5 - 10% of its time.
    ``reset()`` runs in front of each of the two passes.  Returns seconds per iteration of the bare pass."""
    sync()
    # the interpreter's full collections walk every object torch's import left behind (70 - 80 ms each, once
    # every few hundred iterations): park what exists now in the permanent generation, as training loops do
    gc.collect()
    gc.freeze()
    import torch
    KernelClock.enabled = False
    chunk = max(1, steps // 8)
    marks = []
    try:
        if reset:
            reset()
        t0 = time.perf_counter()
        for i in range(steps):
            if i % chunk == 0:                      # one event per chunk: where a one-off stall fell shows afterwards
                marks.append(torch.cuda.Event(enable_timing=True))
                marks[-1].record()
            step()
        marks.append(torch.cuda.Event(enable_timing=True))
        marks[-1].record()
        sync()
        sec = (time.perf_counter() - t0) / steps
    finally:
        KernelClock.enabled = True
    spans = [(a.elapsed_time(b), min(chunk, steps - k * chunk)) for k, (a, b) in enumerate(zip(marks[:-1], marks[1:]))]
    LAST_CHUNKS[:] = [ms / n for ms, n in spans if n == chunk]
    for c in clocks.values():
        c.reset()
    if reset:
        reset()
    for _ in range(min(steps, PHASE_STEPS)):
        step()
    sync()
    gc.unfreeze()
    return sec


# ----------------------------------------------------------------------------------------- C2
def c2_bytes_fwd(R, E, F, s_row=4, mode="src"):
    # (R+1) ptr + E idx + E map lookups + E rows + R output rows  (int64 indices, fp32 data)
    return (R + 1) * 8 + 2 * E * 8 + E * F * s_row + R * F * 4


def c2_bytes_bwd(R, E, F, n_src):
    # E g-rows + E transposed-edge ids + (n_src+1) ptrT + R degrees + n_src output rows
    return E * F * 4 + E * 8 + (n_src + 1) * 8 + R * 4 + n_src * F * 4


def run_c2(args, row_mode=False):
    import torch

    import hiscache_backend as be
    from hiscache.synthetic import power_law_block

    dev = "cuda:0"
    s = args.scale
    R, E, N, F = int(1_000_000 * s), int(20_000_000 * s), int(10_000_000 * s), 256
    ptr, idx = power_law_block(R, E, N, alpha=2.1, max_degree=5000, seed=2)
    ptr, idx = ptr.to(dev), idx.to(dev)
    gen = torch.Generator(device=dev).manual_seed(2)
    feat = torch.randn(N, F, device=dev, generator=gen)
    g = torch.randn(R, F, device=dev, generator=gen)
    if row_mode:
        # reference-exact substitution: 40% of the destination rows carry a cached embedding
        hbuf = 0.5 * torch.randn(R, F, device=dev, generator=gen)
        hmap = torch.where(torch.rand(R, device=dev, generator=gen) < 0.4,
                           torch.arange(R, device=dev), torch.full((R,), -1, device=dev))
    else:
        hist = 0.5 * torch.randn(N, F, device=dev, generator=gen)
        hmap = torch.where(torch.rand(N, device=dev, generator=gen) < 0.4,
                           torch.arange(N, device=dev), torch.full((N,), -1, device=dev))
    feat.requires_grad_(True)
    clk_f, clk_t, clk_b = KernelClock(), KernelClock(), KernelClock()

    def step():
        # the same three launches the autograd Function issues, with a clock on each
        if row_mode:
            out = clk_f(lambda: be._aggr_fwd(be.SUBST_ROW, ptr, idx, feat.detach(), hmap, hbuf, F, None, R))
            tr = clk_t(lambda: be.build_transpose(ptr, idx, hmap, R, N, want_edges=False))
            clk_b(lambda: be._aggr_bwd(ptr, idx, tr, g, hmap, None, feat, False, tuple(hbuf.shape), F, R, N))
        else:
            out = clk_f(lambda: be._aggr_fwd(be.SUBST_SRC, ptr, idx, feat.detach(), hmap, hist, F, None, R))
            # sources that were substituted by a table row get a zero gradient row (their feature row was
            # not read): their edges are left out of the view, as the autograd Function does
            tr = clk_t(lambda: be.build_transpose(ptr, idx, None, R, N, want_edges=False, history_map_src=hmap))
            clk_b(lambda: be._aggr_bwd(ptr, idx, tr, g, None, None, feat, False, None, 0, R, N))
        return out

    for _ in range(args.warmup):
        step()
    sync()
    for c in (clk_f, clk_t, clk_b):
        c.reset()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    sync()
    sec = (time.perf_counter() - t0) / args.steps

    # autograd round trip once, to show the user-level path runs the same kernels
    if row_mode:
        out = be.aggr_forward_history(feat, ptr, idx, hmap, hbuf, F, R)
    else:
        out = be.aggr_forward_source_history(feat, ptr, idx, hmap, hist)
    out.backward(g)
    sync()
    feat.grad = None

    t_f, t_t, t_b = clk_f.mean_ms(), clk_t.mean_ms(), clk_b.mean_ms()
    full_grad = None
    if not row_mode:
        # The same step when the history table wants its gradient too: no source is left out, the view holds all E
        # edges and the backward gathers a gradient row for every one of them (a backward of
        # E*F*4 + E*8 + (N+1)*8 + R*4 + N*F*4 algorithmic bytes).  Timed with the forward beside it, so that the
        # three parts come from the same stretch of the run.
        ck_f, ck_t, ck_b = KernelClock(), KernelClock(), KernelClock()

        def full_step():
            ck_f(lambda: be._aggr_fwd(be.SUBST_SRC, ptr, idx, feat.detach(), hmap, hist, F, None, R))
            tr = ck_t(lambda: be.build_transpose(ptr, idx, None, R, N, want_edges=False))
            ck_b(lambda: be._aggr_bwd(ptr, idx, tr, g, None, None, feat, False, None, 0, R, N))

        for _ in range(args.warmup):
            full_step()
        sync()
        for c in (ck_f, ck_t, ck_b):
            c.reset()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            full_step()
        sync()
        sec_full = (time.perf_counter() - t0) / args.steps
        bytes_b_full = c2_bytes_bwd(R, E, F, N)
        full_grad = {
            "what": "the step with the table's gradient requested: the view holds all %d edges and the backward "
                    "gathers every one of them" % E,
            "ms_per_step": sec_full * 1e3, "edges_per_s": E / sec_full,
            "fwd_ms": ck_f.mean_ms(), "transpose_ms": ck_t.mean_ms(), "bwd_ms": ck_b.mean_ms(),
            "bwd_algorithmic_bytes": bytes_b_full, "bwd_GBps": bytes_b_full / ck_b.mean_ms() / 1e6,
            "bwd_frac": bytes_b_full / ck_b.mean_ms() / 1e6 / HBM_PEAK_GBS,
            "step_algorithmic_bytes": c2_bytes_fwd(R, E, F) + bytes_b_full,
            "step_frac_of_peak": (c2_bytes_fwd(R, E, F) + bytes_b_full) / sec_full / 1e9 / HBM_PEAK_GBS,
        }
    if row_mode:
        n_hist = int((hmap != -1).sum())
        deg = (ptr[1:] - ptr[:-1])
        e_nh = int(deg[hmap == -1].sum())
        bytes_f = (R + 1) * 8 + R * 8 + e_nh * 8 + e_nh * F * 4 + n_hist * F * 4 + R * F * 4
        bytes_b = e_nh * F * 4 + e_nh * 8 + (N + 1) * 8 + R * 4 + N * F * 4 + 2 * n_hist * F * 4
    else:
        bytes_f = c2_bytes_fwd(R, E, F)
        # backward gathers the edges whose source was read from the feature matrix and writes every source row
        e_feat = int((hmap[idx[: int(ptr[R])]] == -1).sum())
        bytes_b = c2_bytes_bwd(R, e_feat, F, N)
    step_bytes = bytes_f + bytes_b
    res = {
        "metric": "aggregated edges/sec (fwd+bwd)",
        "value": E / sec,
        "value_definition": "edges of the forward (%d) per second of the whole step (forward + view + backward); "
                            "the backward of this step gathers kernels.bwd_edges_gathered of them%s"
                            % (E, "" if row_mode else
                               " (substituted sources get zero rows); kernels.full_grad is the step whose backward "
                               "gathers all of them"),
        "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": ("c2row" if row_mode else "c2") +
                   ": history_aggr microbench, R=%d rows, E=%d edges (Zipf 2.1, max deg 5000), %d sources x %d fp32, "
                   "40%% history hits (%s substitution), mean fwd + transpose build + bwd"
                   % (R, E, N, F, "per-row" if row_mode else "per-source")},
        "roofline": {"bound": "hbm",
                     "kernel": "fwd_mean_fast<float,float,4,1,8,%s,0>" % ("false" if row_mode else "true"),
                     "achieved": bytes_f / (t_f * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bytes_f / (t_f * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC["c2row" if row_mode else "c2"] if s == 1.0 else None,
                     "traffic_source": "profiles/aggr_c2_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                                       "this command, scaled by a 4 GiB copy)",
                     "algorithmic_bytes": bytes_f, "launch_ms": t_f},
        "kernels": {
            "fwd_ms": t_f, "fwd_GBps": bytes_f / t_f / 1e6, "fwd_edges_per_s": E / (t_f * 1e-3),
            "transpose_ms": t_t,
            "bwd_ms": t_b, "bwd_GBps": bytes_b / t_b / 1e6, "bwd_edges_per_s": E / (t_b * 1e-3),
            "fwd_plus_bwd_edges_per_s": E / ((t_f + t_b) * 1e-3),
            "fwd_plus_bwd_GBps": (bytes_f + bytes_b) / (t_f + t_b) / 1e6,
            "bwd_edges_gathered": E if row_mode else e_feat,
            # the whole step against the peak: algorithmic bytes of forward + backward over the step time
            # (the transposed-view build is in the time, not in the bytes)
            "step_frac_of_peak": step_bytes / sec / 1e9 / HBM_PEAK_GBS,
        },
    }
    if full_grad is not None:
        res["kernels"]["full_grad"] = full_grad
    return res, dict(R=R, E=E, N=N, F=F)


def run_c2w(args):
    """Weighted (edge_value) aggregation on the C2 block: forward, transposed view with edge slots,
    backward of the input and the SDDMM gradient of the edge values."""
    import torch

    import hiscache_backend as be
    from hiscache.synthetic import power_law_block

    dev = "cuda:0"
    s = args.scale
    R, E, N, F = int(1_000_000 * s), int(20_000_000 * s), int(10_000_000 * s), 256
    ptr, idx = power_law_block(R, E, N, alpha=2.1, max_degree=5000, seed=2)
    ptr, idx = ptr.to(dev), idx.to(dev)
    gen = torch.Generator(device=dev).manual_seed(2)
    H = max(1, int(args.heads))
    if F % H != 0:
        raise SystemExit("--heads must divide %d" % F)
    feat = torch.randn(N, F, device=dev, generator=gen)
    g = torch.randn(R, F, device=dev, generator=gen)
    ev = torch.rand(E, device=dev, generator=gen)
    if H > 1:        # the same bytes seen as H heads of F / H elements with a weight per edge and head
        feat, g = feat.view(N, H, F // H), g.view(R, H, F // H)
        ev = torch.rand(E, H, device=dev, generator=gen)
    clk_f, clk_t, clk_b = KernelClock(), KernelClock(), KernelClock()

    def step():
        clk_f(lambda: be._aggr_fwd(be.SUBST_ROW, ptr, idx, feat, None, None, 0, ev, R))
        tr = clk_t(lambda: be.build_transpose(ptr, idx, None, R, N, want_edges=True))
        clk_b(lambda: be._aggr_bwd(ptr, idx, tr, g, None, ev, feat, True, None, 0, R, N))

    for _ in range(args.warmup):
        step()
    sync()
    for c in (clk_f, clk_t, clk_b):
        c.reset()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    sync()
    sec = (time.perf_counter() - t0) / args.steps
    t_f, t_t, t_b = clk_f.mean_ms(), clk_t.mean_ms(), clk_b.mean_ms()
    bytes_f = (R + 1) * 8 + E * (8 + 4 * H) + E * F * 4 + R * F * 4
    bytes_b = E * F * 4 + E * (4 + 4 + 4 * H) + (N + 1) * 8 + N * F * 4  # input gradient
    bytes_eg = E * (2 * F * 4 + 8 + 4 * H)                                # edge gradient: two rows per edge
    return {
        "metric": "aggregated edges/sec (weighted fwd+bwd+edge_grad)", "value": E / sec, "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c2w: weighted aggregation (edge_value) on the c2 block, R=%d, E=%d, %d sources x %d "
                               "fp32 in %d head(s): fwd + transposed view with edge slots + bwd (input gradient and "
                               "edge gradient)" % (R, E, N, F, H)},
        "roofline": {"bound": "hbm", "kernel": "fwd_mean_fast<float,4,1,8,false,%d>" % (2 if H > 1 else 1),
                     "achieved": bytes_f / (t_f * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bytes_f / (t_f * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes": bytes_f, "launch_ms": t_f},
        "kernels": {"fwd_ms": t_f, "fwd_GBps": bytes_f / (t_f * 1e-3) / 1e9, "transpose_ms": t_t, "bwd_ms": t_b,
                    "bwd_GBps": (bytes_b + bytes_eg) / (t_b * 1e-3) / 1e9},
    }


def cpu_baseline_c2(shape):
    """The same step (forward with per-source substitution, transposed view, backward gather) written in
    C with OpenMP over rows / sources, on a 1/10-size sample, on all the host cores the box grants."""
    import numpy as np

    from hiscache.synthetic import power_law_block
    from oracle import hc_cpu_mt as mt

    R, E, N, F = shape["R"] // 10, shape["E"] // 10, shape["N"] // 10, shape["F"]
    ptr, idx = power_law_block(R, E, N, alpha=2.1, max_degree=5000, seed=2)
    ptr, idx = ptr.numpy(), idx.numpy()
    rng = np.random.default_rng(2)
    feat = rng.standard_normal((N, F), dtype=np.float32)
    hist = 0.5 * rng.standard_normal((N, F), dtype=np.float32)
    hmap = np.where(rng.random(N) < 0.4, np.arange(N), -1).astype(np.int64)
    g = rng.standard_normal((R, F), dtype=np.float32)
    out, gx = np.zeros((R, F), np.float32), np.zeros((N, F), np.float32)
    ptrT, rowT = np.zeros(N + 1, np.int64), np.zeros(E, np.int32)

    def one():
        mt.fwd_mean_src(ptr, idx, feat, hmap, hist, split_above=256, out=out)
        mt.build_transpose(ptr, idx, N, ptrT, rowT, hmap_src=hmap)
        mt.bwd_mean(ptr, ptrT, rowT, g, N, chunk=512, out=gx)

    one()
    one()
    times = []
    t_end = time.perf_counter() + 20.0
    while len(times) < 9 and (len(times) < 3 or time.perf_counter() < t_end):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    tq = torch_spelling_c2(ptr, idx, feat, hist, hmap, g, R, E, N)
    # The headline baseline is the reference semantics spelled with stock PyTorch CPU operators (gather +
    # index_add_), as a PyTorch user would run the step on the host; the C/OpenMP statement of the same step
    # (same sums, same order, what the parity tests check against) rides beside it.
    return {"value": tq["value"], "unit": "edges/s", "cores": tq["threads"], "kind": "port",
            "spelling": "torch_index_add",
            "sample": "1/10-size c2 block (R=%d, E=%d, %d sources x %d fp32), fwd + bwd with PyTorch CPU operators "
                      "(index_select, index_add_, where) on %d threads, median of %d runs"
                      % (R, E, N, F, tq["threads"], tq["runs"]),
            "openmp_c_port": {"value": E / med, "unit": "edges/s", "cores": mt.num_threads(),
                              "sample": "the same block: fwd + transposed view + bwd in C with OpenMP over rows and "
                                        "sources, median of %d runs" % len(times)}}


def torch_spelling_c2(ptr, idx, feat, hist, hmap, g, R, E, N):
    """The same sample through stock PyTorch CPU operators (index_add), the way a PyTorch user would spell
    the step on a CPU: edges/s, median of up to 3 runs."""
    import torch

    from oracle import torch_cpu_path as tp

    torch.set_num_threads(host_threads())
    t = [torch.from_numpy(a) for a in (ptr, idx, feat, hist, hmap, g)]
    ptr, idx, feat, hist, hmap, g = t

    def one():
        tp.aggr_fwd_src(feat, hist, hmap, ptr, idx, R)
        tp.aggr_bwd_src(g, ptr, idx, hmap, N, R)

    one()
    times = []
    t_end = time.perf_counter() + 8.0
    while len(times) < 3 and (not times or time.perf_counter() < t_end):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    times.sort()
    return {"value": E / times[len(times) // 2], "unit": "edges/s", "threads": torch.get_num_threads(),
            "runs": len(times)}


def cpu_baseline_c4(M, F):
    """The fused admission (scores, predicate, ring slots in row order, maps, fp32 -> fp16 row copy) written
    in C with OpenMP over row ranges, on a 1/4-size sample, on all the host cores the box grants."""
    import numpy as np

    from oracle import hc_cpu_mt as mt

    M = M // 4
    cap, Nfull = 2 * M, 4 * M
    rng = np.random.default_rng(4)
    grad = rng.standard_normal((M, F), dtype=np.float32)          # random directions, LogNormal(-3, 1.5) L2 norms
    grad *= (np.exp(rng.normal(-3.0, 1.5, size=(M, 1))) / np.linalg.norm(grad, axis=1, keepdims=True)).astype(np.float32)
    emb = rng.standard_normal((M, F), dtype=np.float32)
    age = rng.integers(0, 21, size=M).astype(np.int32)
    sub_to_full = rng.permutation(Nfull)[:M].astype(np.int64)
    slot = np.where(rng.random(M) < 0.35, rng.permutation(cap)[:M], -1).astype(np.int64)
    table = np.zeros((cap, F), np.uint16)
    full2slot, slot2full = np.full(Nfull, -1, np.int64), np.full(cap, -1, np.int64)
    checkin, header = np.full(cap, -1, np.int64), np.zeros(1, np.int64)

    def one():
        header[0] = 0
        return mt.grad_check_f16(grad, emb, slot, age, sub_to_full, 0.05, 10, table, full2slot, slot2full, checkin,
                                 header, 1)

    one()
    one()
    times = []
    for _ in range(9):
        t0 = time.perf_counter()
        mask, _ = one()
        times.append(time.perf_counter() - t0)
    times.sort()
    return {"value": M / times[4], "unit": "rows/s", "cores": mt.num_threads(), "kind": "port",
            "sample": "%d rows x %d fp32 (1/4 of c4), %d admitted: fused admission into an fp16 ring table in C with "
                      "OpenMP over row ranges (same scores, slots and table bits), median of 9 runs"
                      % (M, F, int(mask.sum()))}


# ----------------------------------------------------------------------------------------- C4
def run_c4(args):
    import torch

    import hiscache_backend as be
    from hiscache.synthetic import lognormal_grads

    dev = "cuda:0"
    s = args.scale
    M, F, cap = int(2_000_000 * s), 256, int(50_000_000 * s)
    gen = torch.Generator(device=dev).manual_seed(4)
    grad = lognormal_grads(M, F, -3.0, 1.5, device=dev, generator=gen)
    emb = torch.randn(M, F, device=dev, generator=gen)
    age = torch.randint(0, 21, (M,), device=dev, generator=gen, dtype=torch.int32)
    Nfull = max(4 * M, cap)
    sub_to_full = torch.randperm(Nfull, device=dev, generator=gen)[:M].contiguous()
    cached = torch.rand(M, device=dev, generator=gen) < 0.35
    slot0 = torch.where(cached, torch.randperm(cap, device=dev, generator=gen)[:M], torch.full((M,), -1, device=dev))
    table = torch.zeros(cap, F, dtype=torch.float16, device=dev)
    full2slot = torch.full((Nfull,), -1, dtype=torch.int64, device=dev)
    slot2full = torch.full((cap,), -1, dtype=torch.int64, device=dev)
    checkin = torch.full((cap,), -1, dtype=torch.int64, device=dev)
    header = torch.zeros(1, dtype=torch.int64, device=dev)
    thres = torch.tensor([0.05], device=dev)
    state = {"A": 0}

    def step():
        header.zero_()
        mask, _ = be.grad_check(grad, emb, slot0, sub_to_full, thres, table, full2slot, slot2full, header, 1,
                                age=age, age_limit=10, checkin=checkin)
        state["mask"] = mask

    sec = timed_steps(step, args.steps, args.warmup)
    A = int(state["mask"].sum())
    # rows whose score sits within 4 ulp of the threshold (a differently ordered sum could flip them)
    score = be.row_scores(grad)
    guard = int(((score.view(torch.int32) - thres.view(torch.int32)).abs() <= 4).sum())
    bytes_ = M * F * 4 + M * 13 + M + A * (F * 4 + F * 2 + 32)
    # the admission threshold of a sampled batch (one block's radix select): us per call, 50 calls replayed
    # back to back as one graph
    from hiscache.util import quantile_threshold
    quantile_us = {}
    side = torch.cuda.Stream()
    for n in (1000, 5800, 10_000, 16_384, 30_000):
        sc = score[:n].contiguous()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            quantile_threshold(sc, 0.9)
            with torch.cuda.graph(graph, stream=side):
                for _ in range(50):
                    quantile_threshold(sc, 0.9)
        torch.cuda.synchronize()
        best = None
        for _ in range(5):
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            graph.replay()
            t1.record()
            torch.cuda.synchronize()
            us = t0.elapsed_time(t1) / 50 * 1e3
            best = us if best is None or us < best else best
        quantile_us[str(n)] = round(best, 2)
    return {
        "quantile_threshold_us_per_call": quantile_us,
        "metric": "grad_check admission rows/sec", "value": M / sec, "unit": "rows/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c4: grad_check microbench, %d rows x %d fp32 grads (lognormal norms), ages in [0,20], "
                               "thres 0.05, age limit 10, fp16 table %d x %d; admitted %d; %d rows within 4 ulp of the "
                               "threshold" % (M, F, cap, F, A, guard)},
        "roofline": {"bound": "hbm", "kernel": "gc_pass1+gc_pass2+gc_pass3_ring", "achieved": bytes_ / sec / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bytes_ / sec / 1e9 / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC["c4"] if s == 1.0 else None, "algorithmic_bytes": bytes_},
    }


# ----------------------------------------------------------------------------------------- C3
def c3_batched_layer(args, samples=None):
    """The papers100M-shaped history layer for about 800 batches side by side (about 20 M edges): forward with
    per-row substitution from an fp16 row-aligned buffer, transposed-view build, backward, fused admission of the
    produced rows into an fp16 ring.  The roofline fraction counts the algorithmic bytes of forward, backward and
    admission over the time of all four steps (the transposed-view build is in the time, not in the bytes)."""
    import numpy as np
    import torch

    import hiscache_backend as be
    from hiscache.synthetic import batched_history_layer, direct_power_law_batch, lognormal_grads

    dev = "cuda:0"
    s = args.scale
    N, H = int(111_000_000 * s), 256
    if samples is None:
        samples = [direct_power_law_batch(N, 1000, [15, 10, 5], 2.0, 30 + i, degree_scale=2.6) for i in range(8)]
    gen = torch.Generator(device=dev).manual_seed(33)
    ptr_h, idx_h, R, E, Nsrc = batched_history_layer(samples[:8], int(20_000_000 * s))
    ptr, idx = torch.from_numpy(ptr_h).to(dev), torch.from_numpy(idx_h).to(dev)
    x = torch.randn(Nsrc, H, device=dev, generator=gen)
    hbuf = (0.5 * torch.randn(R, H, device=dev, generator=gen)).half()
    hmap = torch.where(torch.rand(R, device=dev, generator=gen) < 0.35, torch.arange(R, device=dev),
                       torch.full((R,), -1, device=dev))
    g = torch.randn(R, H, device=dev, generator=gen)
    grad = lognormal_grads(R, H, -3.0, 1.5, device=dev, generator=gen)
    emb = torch.randn(R, H, device=dev, generator=gen)
    cap = max(R, 1 << 20)
    table = torch.zeros(cap, H, dtype=torch.float16, device=dev)
    f2s = torch.full((2 * R,), -1, dtype=torch.int64, device=dev)
    s2f = torch.full((cap,), -1, dtype=torch.int64, device=dev)
    chk = torch.full((cap,), -1, dtype=torch.int64, device=dev)
    hdr = torch.zeros(1, dtype=torch.int64, device=dev)
    sub_to_full = torch.randperm(2 * R, device=dev, generator=gen)[:R].contiguous()
    thr = torch.tensor([0.05], device=dev)
    cf, ct, cb, cg, cv = KernelClock(), KernelClock(), KernelClock(), KernelClock(), KernelClock()
    st = {}
    # the view of the whole block with nothing left out, as a loader emits it with a batch (built once, outside
    # the time): the backward over it steps over the history rows' edges in the kernel; reported beside the figures
    # of the step above, whose time includes the view it builds
    shared_view = be.build_batch_view(ptr, idx, R, Nsrc)

    def kstep():
        cf(lambda: be._aggr_fwd(be.SUBST_ROW, ptr, idx, x, hmap, hbuf, H, None, R))
        tr = ct(lambda: be.build_transpose(ptr, idx, hmap, R, Nsrc, want_edges=False))
        # as in the training iteration, the cached embeddings need no gradient: no grad_hbuf is written
        cb(lambda: be._aggr_bwd(ptr, idx, tr, g, hmap, None, x, False, (R, H), H, R, Nsrc, want_hist_grad=False))
        hdr.zero_()
        st["mask"] = cg(lambda: be.grad_check(grad, emb, hmap, sub_to_full, thr, table, f2s, s2f, hdr, 1,
                                              checkin=chk))[0]
        cv(lambda: be._aggr_bwd_batch_view(ptr, shared_view, g, hmap, None, H, R, Nsrc, want_hist_grad=False))

    for _ in range(args.warmup):
        kstep()
    sync()
    for c in (cf, ct, cb, cg, cv):
        c.reset()
    for _ in range(args.steps):
        kstep()
    sync()
    t_f, t_t, t_b, t_g = cf.mean_ms(), ct.mean_ms(), cb.mean_ms(), cg.mean_ms()
    n_hist = int((hmap != -1).sum())
    deg = ptr[1:] - ptr[:-1]
    e_nh = int(deg[hmap == -1].sum())
    A = int(st["mask"].sum())
    bytes_f = (R + 1) * 8 + R * 8 + e_nh * 8 + e_nh * H * 4 + n_hist * H * 2 + R * H * 4
    bytes_b = e_nh * H * 4 + e_nh * 8 + (Nsrc + 1) * 8 + R * 4 + Nsrc * H * 4
    bytes_g = R * H * 4 + R * 13 + R + A * (H * 4 + H * 2 + 32)
    tot_b, tot_t = bytes_f + bytes_b + bytes_g, (t_f + t_t + t_b + t_g) * 1e-3
    detail = {
        "rows": R, "edges": E, "sources": Nsrc, "history_rows": n_hist, "admitted": A,
        "fwd_ms": t_f, "transpose_ms": t_t, "bwd_ms": t_b, "grad_check_ms": t_g,
        "fwd_GBps": bytes_f / t_f / 1e6, "bwd_GBps": bytes_b / t_b / 1e6, "grad_check_GBps": bytes_g / t_g / 1e6,
        "edges_per_s_fwd_bwd": E / ((t_f + t_t + t_b) * 1e-3),
        "algorithmic_bytes": tot_b, "ms": tot_t * 1e3, "frac": tot_b / tot_t / 1e9 / HBM_PEAK_GBS,
        "traffic": MEASURED_TRAFFIC["c3_batched"] if s == 1.0 else None,
        # the same time against the bytes that the counters saw cross the memory interface (the gradient rows of
        # the backward are partly served by the caches, so this is the smaller figure)
        "frac_by_counters": (MEASURED_TRAFFIC["c3_batched"] / tot_t / 1e9 / HBM_PEAK_GBS) if s == 1.0 else None,
        # beside it: the same layer when the batch comes with its view (no build in the step; backward over the
        # whole block's view)
        "bwd_over_emitted_view_ms": cv.mean_ms(),
        "frac_with_emitted_view": tot_b / ((t_f + cv.mean_ms() + t_g) * 1e-3) / 1e9 / HBM_PEAK_GBS,
    }
    roofline = {"bound": "hbm",
                "kernel": "fwd_mean_fast + transposed view + bwd_mean_fast + gc_pass1..3 (batched history layer)",
                "achieved": tot_b / tot_t / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": tot_b / tot_t / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes": tot_b}
    return {"detail": detail, "roofline": roofline}


def pooled_store_class(pool_rows):
    """PinnedFeatureStore over a pinned POOL of ``pool_rows`` rows that stands for a feature matrix too large
    for this host: node ids are folded into the pool.  Every read shifts the folding, so that the batches of
    this benchmark touch new pool rows each time, as the batches of a real epoch do (repeated reads of the
    same host rows are served from the GPU's caches: 40 us instead of 640 us for a 46 MB read).  For
    pre-generated batches the folded ids are worked out when the batch is made (``prefold``): the folding is
    the benchmark's stand-in, not part of the iteration."""
    from hiscache import PinnedFeatureStore

    class PooledStore(PinnedFeatureStore):
        reads = 0
        folded = None

        def prefold(self, batches):
            self.folded = {id(b.sub_to_full): (b.sub_to_full, (b.sub_to_full + (k + 1) * 1_000_003) % pool_rows)
                           for k, b in enumerate(batches)}

        def fold(self, ids):
            hit = self.folded.get(id(ids)) if self.folded else None
            if hit is not None and hit[0] is ids:
                return hit[1]
            self.reads += 1
            return (ids + self.reads * 1_000_003) % pool_rows

        def _host_ids(self, ids):
            return self.fold(ids)

    return PooledStore




def run_c3(args, with_batched=True):
    """papers100M-shaped training iteration (one GPU's share at its real batch shape) and a batched
    variant of its history layer (many batches side by side) for the kernels' asymptotic rate."""
    import numpy as np
    import torch

    import hiscache_backend as be
    from hiscache import HistorySAGE, PinnedFeatureStore, RingHistoryCache, make_config, prefer_low_latency_gemm
    from hiscache.synthetic import direct_power_law_batch, make_batch

    dev = "cuda:0"
    s = args.scale
    N, Fin, H, C = int(111_000_000 * s), 128, 256, 172
    fanout, n_seed, L = [15, 10, 5], 1000, 3
    pool_rows = min(N, 16_000_000)

    PooledStore = pooled_store_class(pool_rows)

    gen = torch.Generator(device=dev).manual_seed(3)
    pinned = torch.empty((pool_rows, Fin), dtype=torch.float32, pin_memory=True)
    chunk = 2_000_000
    for lo in range(0, pool_rows, chunk):
        hi = min(pool_rows, lo + chunk)
        pinned[lo:hi].copy_(torch.randn(hi - lo, Fin, device=dev, generator=gen))
    if args.features_in_hbm:
        pinned = pinned.to(dev)
    store = PooledStore(pinned, device=dev, prefetch_cus=args.prefetch_cus if args.prefetch else 0)
    cache = RingHistoryCache(store, N, Fin, H, capacity=N, num_layers=L, table_dtype=torch.float16,
                             thres=0.05, age_limit=AGE_LIMIT_ITERS, device=dev)
    # about 35% of the nodes start with a cached embedding
    hit = torch.nonzero(torch.rand(N, device=dev, generator=gen) < 0.35).view(-1)
    cache.preload(hit)
    cache.table.normal_(0.0, 0.5, generator=gen) if N <= 20_000_000 else cache.table[:hit.numel()].normal_(0.0, 0.5)
    cfg = make_config(Fin, C, H, L, device=dev)
    torch.manual_seed(3)
    prefer_low_latency_gemm()                                            # what get_model() does by default
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache).to(dev)
    model.train()
    # one multi-tensor launch per step
    opt = torch.optim.Adam(model.parameters(), lr=1e-3, fused=True, capturable=bool(args.recorded))
    recorded = None
    if args.recorded:
        # (a read inside a recording keeps the pooled store's folding offset of the moment it was recorded; the
        # batches differ, so the pool rows read still differ from replay to replay)
        from hiscache import RecordedIteration
        recorded = RecordedIteration(model, cache, opt, L)
    class FoldedLabels:
        """Labels of a huge id space folded into a small table."""
        base = np.random.default_rng(3).integers(0, C, size=1 << 20)

        def __getitem__(self, ids):
            return self.base[np.asarray(ids) % self.base.size]

    labels = FoldedLabels()

    # One batch per iteration, none reused: a batch that comes back finds the 1-hop nodes it admitted last
    # time in the cache, the used masks prune everything below them and no feature row is read at all.
    n_pre = min(args.warmup + args.steps + min(args.steps, PHASE_STEPS) + 1, 640)   # none reused, see time_iterations
    samples = [direct_power_law_batch(N, n_seed, fanout, 2.0, 30 + i, degree_scale=2.6) for i in range(n_pre)]
    batches = []
    for smp in samples:
        # a batch comes with the transposed view of its CSR, as the loader emits it (--no-batch-view: every
        # layer's backward builds its own)
        batches.append(make_batch(smp, labels, dev, emit_view=not args.no_batch_view))
    store.prefold(batches)
    ev = {k: KernelClock() for k in ("load", "forward", "backward", "step", "update")}
    state = {"it": 0}
    sampled = {"sampler": None, "pending": None, "ahead": [], "shapes": [], "wait_s": 0.0, "E_graph": 0}
    if args.with_sampler:
        # batches come from the device sampler over a graph of the same size held in HBM; batch i+1 is
        # sampled on the sampler's side stream while batch i trains
        from hiscache import NeighborSampler
        indptr, indices = device_power_law_graph(N, 14.5, dev, gen)
        sampled["E_graph"] = indices.numel()
        if args.hot_fraction > 0 and not args.features_in_hbm:
            # hotness = incoming edges (what a pre-sampling pass of the reference's preprocessing counts)
            k = min(N, int(N * args.hot_fraction))
            counts = torch.bincount(indices, minlength=N)
            hot_ids = torch.argsort(counts, descending=True)[:k].contiguous()
            del counts
            store.set_hot_rows(hot_ids, num_nodes=N)
            del hot_ids
        sampled["sampler"] = NeighborSampler(indptr, indices, fanout, seed=3, device=dev, validate=False,
                                             emit_view=not args.no_batch_view,
                                             replay_slots=max(args.sampler_replay, args.prefetch_depth + 2)
                                             if args.sampler_replay else 0)
        del indptr, indices
        seed_pool = torch.randperm(N, device=dev, generator=gen)[: n_seed * 1024].view(1024, n_seed).contiguous()
        sampled["pending"] = sampled["sampler"].sample_async(seed_pool[0])

    def sampled_batch(i):
        """Batch i from the sampler (waits only if its sampling is not finished yet); batch i + 1 is started."""
        t1 = time.perf_counter()
        b = sampled["pending"].get()
        sampled["wait_s"] += time.perf_counter() - t1
        b.y = seed_pool[i % 1024] % C
        sampled["pending"] = sampled["sampler"].sample_async(seed_pool[(i + 1) % 1024])
        sampled["shapes"].append(b.num_node_in_layer.tolist() + [b.idx.numel()])
        return b

    def next_batch():
        i = state["it"] - 1
        if sampled["sampler"] is None:
            return batches[i % n_pre]
        if not args.prefetch:
            return sampled_batch(i)
        # batch i was taken from the sampler --prefetch-depth iterations ago, when its feature read started
        if not sampled["ahead"]:
            return sampled_batch(i)
        return sampled["ahead"].pop(0)

    def start_prefetch():
        """The host-link read of the next batch (of the next --prefetch-depth batches), under the masks of the
        cache's present state (--prefetch-all: every row), runs beside this batch's forward and backward."""
        if sampled["sampler"] is None:
            for d in range(args.prefetch_depth):
                nb = batches[(state["it"] + d) % n_pre]
                if getattr(nb, "prefetched_x", None) is None:
                    read_ahead(nb)
            return
        while len(sampled["ahead"]) < args.prefetch_depth:
            nxt = sampled_batch(state["it"] + len(sampled["ahead"]))
            read_ahead(nxt)
            sampled["ahead"].append(nxt)

    def read_ahead(nb):
        if recorded is not None and not args.prefetch_all:
            recorded.prefetch(nb)          # the rows go straight into the array that the batch's recording reads
        else:
            cache.prefetch(nb, speculative=not args.prefetch_all)

    def step():
        state["it"] += 1
        b = next_batch()
        if recorded is not None:
            start_prefetch()                                   # the next batch's rows, beside this replay
            ev["load"](lambda: recorded(b, state["it"]))       # the whole iteration is one replay
            return
        ev["load"](lambda: cache.lookup_and_load(b, L))
        if args.prefetch:
            start_prefetch()
        out = ev["forward"](lambda: model(b))
        loss = torch.nn.functional.nll_loss(out, b.y)
        opt.zero_grad(set_to_none=True)
        ev["backward"](lambda: backward_on_this_thread(loss))
        ev["step"](lambda: opt.step())
        ev["update"](lambda: cache.update_history(b, state["it"]))

    if args.prefetch:
        # the read-ahead only runs beside the compute when the compute is on a stream of its own: the
        # default stream and the read's CU-limited stream wait for each other
        # of a few streams, the one that the reads slow down least (and on another hardware queue than the sampler's)
        compute = store.quiet_stream(apart_from=[sampled["sampler"].stream()] if args.with_sampler else [])
        compute.wait_stream(torch.cuda.current_stream())
        torch.cuda.set_stream(compute)
    for _ in range(args.warmup):
        step()

    def reset():
        sampled["shapes"], sampled["wait_s"] = [], 0.0

    sec = time_iterations(step, args.steps, ev, reset)
    torch.cuda.set_stream(torch.cuda.default_stream())
    if sampled["sampler"] is not None:
        sampled["pending"].get()
        m = np.mean(np.asarray(sampled["shapes"], dtype=np.float64), axis=0)
        shape = {"n0": int(m[0]), "n1": int(m[1]), "n2": int(m[2]), "n3": int(m[3]), "edges": int(m[4]),
                 "sampled_on_device_from_graph_edges": sampled["E_graph"],
                 "wait_for_sampler_ms": 1e3 * sampled["wait_s"] / max(1, len(sampled["shapes"]))}
    else:
        shape = {k: int(np.mean([int(x["num_node_in_layer"][i]) for x in samples])) for i, k in enumerate(("n0", "n1", "n2", "n3"))}
        shape["edges"] = int(np.mean([x["idx"].size for x in samples]))

    batched = c3_batched_layer(args, samples) if with_batched else {"detail": None, "roofline": None}
    rec_info = None
    if recorded is not None:
        rec_info = {"replays": recorded.replays, "unrecorded": recorded.unrecorded,
                    "shapes": {str(k): v[:2] for k, v in recorded.shapes().items()}}
    return {
        "recorded": rec_info,
        "metric": "papers100M-shaped iteration ms (1 GPU)", "value": sec * 1e3, "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c3: papers100M-shaped, %d nodes, 3-layer SAGE hidden 256, fanout [15,10,5], batch 1000, "
                               "fp16 history table %d x 256 (about 35%% of nodes cached), features 128-dim fp32 in a "
                               "%s of %d rows; mean batch %s"
                               % (N, N, "device-memory pool" if args.features_in_hbm else "pinned host pool read zero-copy",
                                  pool_rows, shape)},
        "phases_ms": {k: c.mean_ms() for k, c in ev.items()},
        "phases_host_enqueue_ms": {k: c.mean_cpu_ms() for k, c in ev.items()},
        "ms_per_chunk_of_steps": chunk_figures(),
        "feature_store": "device memory" if args.features_in_hbm else "pinned host memory, read zero-copy",
        "transposed_view": "built in backward" if args.no_batch_view else "emitted with the batch",
        "feature_rows_read_last_batch": int(cache.used_masks[0].sum()),
        "feature_rows_in_device_memory": 0 if store.hot_rows is None else int(store.hot_rows.shape[0]),
        "feature_rows_over_host_link_last_read": None if store.last_cold is None else int(store.last_cold.sum()),
        "cached_1hop_fraction_last_batch": float((cache.sub2embed != -1).float().mean()),
        "batched_history_layer": batched["detail"],
        "roofline": batched["roofline"],
    }


# ----------------------------------------------------------------------------------------- C5
def run_c5(args):
    """mag240M-shaped heterogeneous RGCN iteration: one GPU's share at its real batch shape."""
    import numpy as np
    import torch

    from hiscache import HistoryRGCN, PinnedFeatureStore, RingHistoryCache, make_config, prefer_low_latency_gemm
    from hiscache.synthetic import direct_power_law_batch, make_batch

    dev = "cuda:0"
    s = args.scale
    n_paper, n_author, n_inst = int(122_000_000 * s), int(122_000_000 * s), max(1, int(26_000 * s))
    N = n_paper + n_author + n_inst
    Fin, H, C, K, L = 768, 256, 153, 5, 2
    fanout, n_seed = [25, 15], 1000
    pool_rows = min(N, 4_000_000)

    PooledStore = pooled_store_class(pool_rows)

    gen = torch.Generator(device=dev).manual_seed(5)
    pinned = torch.empty((pool_rows, Fin), dtype=torch.float16, pin_memory=True)
    chunk = 500_000
    for lo in range(0, pool_rows, chunk):
        hi = min(pool_rows, lo + chunk)
        pinned[lo:hi].copy_(torch.randn(hi - lo, Fin, device=dev, generator=gen).half())
    store = PooledStore(pinned, device=dev, out_dtype=torch.float16,
                        prefetch_cus=args.prefetch_cus if args.prefetch else 0)
    cache = RingHistoryCache(store, N, Fin, H, capacity=N, num_layers=L, table_dtype=torch.float16, thres=0.05,
                             age_limit=AGE_LIMIT_ITERS, device=dev)
    hit = torch.nonzero(torch.rand(N, device=dev, generator=gen) < 0.35).view(-1)
    cache.preload(hit)
    del hit
    cfg = make_config(Fin, C, H, L, device=dev, model_type="rgcn", num_rel=K, name="rmag240m")
    torch.manual_seed(5)
    # relation of an edge from the node types of (destination, source): paper-cites-paper,
    # paper<-author, author<-paper, author<-institution, institution<-author
    pair_to_rel = [[0, 1, 0], [2, 0, 3], [0, 4, 0]]
    prefer_low_latency_gemm()                                            # what get_model() does by default
    model = HistoryRGCN(Fin, H, C, L, 0.0, "CSR_Layer", cfg, cache, num_rel=K, dataset_name="rmag240m",
                        type_bounds=[n_paper, n_paper + n_author], pair_to_rel=pair_to_rel).to(dev)
    model.train()
    # one multi-tensor launch per step
    opt = torch.optim.Adam(model.parameters(), lr=1e-3, fused=True, capturable=bool(args.recorded))
    recorded = None
    if args.recorded:
        from hiscache import RecordedIteration
        recorded = RecordedIteration(model, cache, opt, L)

    class FoldedLabels:
        base = np.random.default_rng(5).integers(0, C, size=1 << 20)

        def __getitem__(self, ids):
            return self.base[np.asarray(ids) % self.base.size]

    n_pre = min(args.warmup + args.steps + min(args.steps, PHASE_STEPS) + 1, 640)   # one batch per iteration, none reused
    samples = [direct_power_law_batch(N, n_seed, fanout, 2.0, 50 + i, degree_scale=1.25) for i in range(n_pre)]
    # a batch comes with the transposed view of its CSR (and the view's edge slots, which the relational
    # layer reads), as the loader emits it (--no-batch-view: backward builds the view of the regrouped block)
    batches = [make_batch(smp, FoldedLabels(), dev, emit_view=not args.no_batch_view, view_edges=True)
               for smp in samples]
    store.prefold(batches)
    ev = {k: KernelClock() for k in ("load", "forward", "backward", "step", "update")}
    state = {"it": 0}

    def step():
        b = batches[state["it"] % n_pre]
        state["it"] += 1
        if recorded is not None:
            if args.prefetch:
                recorded.prefetch(batches[state["it"] % n_pre])
            ev["load"](lambda: recorded(b, state["it"]))       # the whole iteration is one replay
            return
        ev["load"](lambda: cache.lookup_and_load(b, L))
        if args.prefetch:             # the next batch's host-link read runs under this batch's compute
            cache.prefetch(batches[state["it"] % n_pre], speculative=not args.prefetch_all)
        out = ev["forward"](lambda: model(b))
        loss = torch.nn.functional.nll_loss(out, b.y)
        opt.zero_grad(set_to_none=True)
        ev["backward"](lambda: backward_on_this_thread(loss))
        ev["step"](lambda: opt.step())
        ev["update"](lambda: cache.update_history(b, state["it"]))

    if args.prefetch:                 # see run_c3: the read-ahead needs the compute on a stream of its own
        compute = store.quiet_stream()
        compute.wait_stream(torch.cuda.current_stream())
        torch.cuda.set_stream(compute)
    for _ in range(args.warmup):
        step()
    sec = time_iterations(step, args.steps, ev)
    torch.cuda.set_stream(torch.cuda.default_stream())
    shape = {k: int(np.mean([int(x["num_node_in_layer"][i]) for x in samples])) for i, k in enumerate(("n0", "n1", "n2"))}
    shape["edges"] = int(np.mean([x["idx"].size for x in samples]))
    return {
        "recorded": None if recorded is None else {"replays": recorded.replays, "unrecorded": recorded.unrecorded,
                                                   "shapes": {str(k): v[:2] for k, v in recorded.shapes().items()}},
        "metric": "mag240M-shaped RGCN iteration ms (1 GPU)", "value": sec * 1e3, "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "c5: mag240M-shaped, %d nodes of 3 types, 5 relations from node-type pairs, 2-layer RGCN "
                               "hidden 256, fanout [25,15], batch 1000, fp16 history table %d x 256 (about 35%% cached), "
                               "features 768-dim fp16 in a pinned host pool of %d rows read zero-copy; mean batch %s"
                               % (N, N, pool_rows, shape)},
        "phases_ms": {k: c.mean_ms() for k, c in ev.items()},
        "phases_host_enqueue_ms": {k: c.mean_cpu_ms() for k, c in ev.items()},
        "ms_per_chunk_of_steps": chunk_figures(),
        "transposed_view": "built in backward" if args.no_batch_view else "emitted with the batch",
        "feature_rows_read_last_batch": int(cache.used_masks[0].sum()),
        "feature_rows_in_device_memory": 0 if store.hot_rows is None else int(store.hot_rows.shape[0]),
        "feature_rows_over_host_link_last_read": None if store.last_cold is None else int(store.last_cold.sum()),
        "cached_1hop_fraction_last_batch": float((cache.sub2embed != -1).float().mean()),
    }


def run_c1(args):
    """The CPU-runnable plumbing configuration (`configs[0]`): uniform graph of 100 k nodes, mean out-degree 15,
    128-dim fp32 features, 10 classes, 2-layer SAGE hidden 128, 1000 seeds, fanout [10, 5], fp32 history table
    100 k x 128 with a random 30% of the nodes cached.  Per-iteration time of sampling (one batch ahead, view
    emitted) -> lookup_and_load -> forward / backward -> optimizer -> admission on the GPU, and of the same
    iteration with stock PyTorch CPU operators over the same batches (`oracle/torch_cpu_path.py`)."""
    import copy

    import numpy as np
    import torch

    from hiscache import HistorySAGE, NeighborSampler, PinnedFeatureStore, RingHistoryCache, make_config, prefer_low_latency_gemm
    from hiscache.synthetic import uniform_graph

    dev = "cuda:0"
    N, Fin, H, C, L, n_seed, fanout, rate = 100_000, 128, 128, 10, 2, 1000, [10, 5], 0.5
    rng = np.random.default_rng(1)
    torch.manual_seed(1)
    indptr, indices = uniform_graph(N, 15, 1)
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    labels = torch.from_numpy(rng.integers(0, C, size=N))
    cached = torch.from_numpy(rng.permutation(N)[: int(0.3 * N)].copy())
    rows = torch.from_numpy(rng.standard_normal((cached.numel(), H)).astype(np.float32))
    cache = RingHistoryCache(PinnedFeatureStore(feats, device=dev), N, Fin, H, capacity=N, num_layers=L,
                             table_dtype=torch.float32, rate=rate, age_limit=AGE_LIMIT_ITERS, device=dev)
    cache.preload(cached.to(dev), rows.to(dev))
    prefer_low_latency_gemm()
    model = HistorySAGE(Fin, H, C, L, 0.0, "CSR_Layer", make_config(Fin, C, H, L, device=dev), cache).to(dev)
    model.train()
    cpu_model = None
    if not args.no_cpu_baseline:
        table, model.table = model.table, None
        cpu_model = copy.deepcopy(model).cpu()
        model.table = table
    opt = torch.optim.Adam(model.parameters(), lr=1e-3, fused=True, capturable=bool(args.recorded))
    recorded = None
    if args.recorded:
        from hiscache import RecordedIteration
        recorded = RecordedIteration(model, cache, opt, L)
    sampler = NeighborSampler(indptr, indices, fanout, labels=labels, seed=1, device=dev, validate=False,
                              emit_view=not args.no_batch_view, replay_slots=args.sampler_replay)
    gen = torch.Generator(device=dev).manual_seed(1)
    seed_pool = torch.randperm(N, device=dev, generator=gen)[: n_seed * 64].view(64, n_seed).contiguous()
    ev = {k: KernelClock() for k in ("load", "forward", "backward", "step", "update")}
    state = {"it": 0, "pending": sampler.sample_async(seed_pool[0]), "shapes": [], "kept": []}

    def step():
        state["it"] += 1
        b = state["pending"].get()
        state["pending"] = sampler.sample_async(seed_pool[state["it"] % 64])
        state["shapes"].append(b.num_node_in_layer.tolist() + [b.idx.numel()])
        if len(state["kept"]) < 8:                  # copies: a replayed sampler overwrites a batch's arrays later
            state["kept"].append(types.SimpleNamespace(ptr=b.ptr.clone(), idx=b.idx.clone(), y=b.y.clone(),
                                                       sub_to_full=b.sub_to_full.clone(),
                                                       num_node_in_layer=b.num_node_in_layer.clone()))
        if recorded is not None:
            ev["load"](lambda: recorded(b, state["it"]))      # the whole iteration is one replay
            return
        ev["load"](lambda: cache.lookup_and_load(b, L))
        out = ev["forward"](lambda: model(b))
        loss = torch.nn.functional.nll_loss(out, b.y)
        opt.zero_grad(set_to_none=True)
        ev["backward"](lambda: backward_on_this_thread(loss))
        ev["step"](lambda: opt.step())
        ev["update"](lambda: cache.update_history(b, state["it"]))

    for _ in range(args.warmup):
        step()

    def reset():
        state["shapes"] = []

    sec = time_iterations(step, args.steps, ev, reset)
    state["pending"].get()
    m = np.mean(np.asarray(state["shapes"], dtype=np.float64), axis=0)
    res = {
        "metric": "plumbing-configuration iteration ms (1 GPU)", "value": sec * 1e3, "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c1: 100000 nodes, mean out-degree 15, 2-layer SAGE hidden 128, fanout [10,5], batch 1000, "
                               "fp32 history table 100000 x 128 (30%% of the nodes cached), features 128-dim fp32 in pinned "
                               "host memory read zero-copy, batches from the device sampler; mean batch n0 %d, n1 %d, "
                               "n2 %d, %d edges" % tuple(int(v) for v in m)},
        "phases_ms": {k: c.mean_ms() for k, c in ev.items()},
        "phases_host_enqueue_ms": {k: c.mean_cpu_ms() for k, c in ev.items()},
        "ms_per_chunk_of_steps": chunk_figures(),
        "transposed_view": "built in backward" if args.no_batch_view else "emitted with the batch",
    }
    if recorded is not None:
        res["recorded"] = {"replays": recorded.replays, "unrecorded": recorded.unrecorded,
                           "shapes": {str(k): v[:2] for k, v in recorded.shapes().items()}}
    if cpu_model is not None:
        # the same iteration with stock PyTorch CPU operators, over batches the GPU loop trained on
        from oracle import torch_cpu_path as tp
        cpu_model.train()
        cpu_opt = torch.optim.Adam(cpu_model.parameters(), lr=1e-3)
        ring = tp.ring_state(N, N, H)
        ring["table"][: cached.numel()] = rows
        ring["f2s"][cached] = torch.arange(cached.numel())
        ring["s2f"][: cached.numel()] = cached
        ring["checkin"][: cached.numel()] = 0
        ring["header"] = cached.numel() % N
        cpu_batches = [dict(ptr=b.ptr.cpu().numpy(), idx=b.idx.cpu().numpy(), sub_to_full=b.sub_to_full.cpu().numpy(),
                            num_node_in_layer=b.num_node_in_layer.numpy(), y=b.y.cpu()) for b in state["kept"]]
        torch.set_num_threads(host_threads())
        tp.sage_iteration(cpu_model, cpu_opt, cpu_batches[0], feats, ring, 1, rate)          # warm-up
        t0 = time.perf_counter()
        for k, cb in enumerate(cpu_batches[1:], start=2):
            tp.sage_iteration(cpu_model, cpu_opt, cb, feats, ring, k, rate)
        cpu_ms = (time.perf_counter() - t0) / max(len(cpu_batches) - 1, 1) * 1e3
        res["cpu_baseline"] = {"value": cpu_ms, "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "%d iterations of the same configuration over batches the GPU loop trained on, "
                                         "stock PyTorch CPU operators (index_add aggregation, torch.quantile admission; "
                                         "used masks by the sequential C statement)" % max(len(cpu_batches) - 1, 1)}
    return res


def run_layer(args):
    """The dense side of a sampled layer: weight gradients (hc_weight_grad against the library GEMM and its
    slab-batched spelling) and the bias + batch norm + ReLU epilogue (hc_bn_relu against torch's operators), at
    the row counts of the papers100M-shaped layers and of the sampler-fed loop.  Kernel time by HIP events; every
    call is long enough for the device, not the host, to set the pace."""
    import torch
    import torch.nn.functional as Fn

    import hiscache_backend as be
    from hiscache import history_model as hm, prefer_low_latency_gemm

    prefer_low_latency_gemm()
    dev = "cuda:0"

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.steps * 1e3

    H = 256
    wg, bn = [], []
    for n, F in ((5_800, 256), (25_800, 128), (25_800, 256), (55_000, 128), (55_000, 256), (89_000, 128)):
        g = torch.randn(n, H, device=dev)
        x0, x1 = torch.randn(n, F, device=dev), torch.randn(n, F, device=dev)
        t_k = timed(lambda: be.weight_grad(g, x0, x1))
        t_mm = timed(lambda: (g.t() @ x0, g.t() @ x1))
        t_sl = timed(lambda: (hm._weight_grad(g, x0), hm._weight_grad(g, x1)))
        flop = 2 * 2.0 * n * H * F
        wg.append({"rows": n, "H": H, "F": F, "hc_weight_grad_us": t_k, "hc_weight_grad_TFLOPs": flop / t_k / 1e6,
                   "library_gemm_us": t_mm, "slab_batched_gemm_us": t_sl})
    for n in (5_800, 25_800, 55_000):
        z = torch.randn(n, H, device=dev)
        bias, gamma, beta = (torch.randn(H, device=dev) for _ in range(3))
        rm, rv = torch.zeros(H, device=dev), torch.ones(H, device=dev)
        dy = torch.randn(n, H, device=dev)

        def ours():
            zi = z.requires_grad_(True)
            y = be.bias_bn_relu(zi, bias, gamma, beta, rm, rv, 0.1, 1e-5)
            torch.autograd.grad(y, zi, dy)

        def torch_ops():
            zi = z.requires_grad_(True)
            y = Fn.relu(Fn.batch_norm(zi + bias, rm, rv, gamma, beta, True, 0.1, 1e-5))
            torch.autograd.grad(y, zi, dy)

        bn.append({"rows": n, "C": H, "hc_bn_relu_fwd_bwd_us": timed(ours), "torch_fwd_bwd_us": timed(torch_ops)})
    big = wg[-1]
    return {"metric": "weight-gradient TFLOP/s (fp32, two operands, 89 000 rows)", "value": big["hc_weight_grad_TFLOPs"],
            "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": big["hc_weight_grad_us"] / 1e3, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "layer: weight gradients g^T x (g [n, 256], two operands [n, F]) and bias + batch "
                                   "norm + ReLU forward/backward of [n, 256], n = rows of sampled layers"},
            "roofline": {"bound": "mfma", "kernel": "wg_partial + wg_reduce", "achieved": big["hc_weight_grad_TFLOPs"],
                         "peak": 157.3, "unit": "TFLOP/s", "frac": big["hc_weight_grad_TFLOPs"] / 157.3, "traffic": None},
            "weight_grad": wg, "bn_relu": bn}


def run_c3b(args):
    """The batched papers100M-shaped history layer measured several times in one process, its tensors freed
    and allocated again between the measurements: the spread of its figure with where the allocations land."""
    import gc

    import torch

    reps = []
    for _ in range(max(1, args.reps)):
        d = c3_batched_layer(args)["detail"]
        reps.append({k: d[k] for k in ("fwd_ms", "transpose_ms", "bwd_ms", "grad_check_ms", "ms", "frac")})
        gc.collect()
        torch.cuda.empty_cache()
    fr = sorted(r["frac"] for r in reps)
    return {"metric": "batched history layer, fraction of 8 TB/s (median over re-allocations)", "value": fr[len(fr) // 2],
            "unit": "fraction of HBM peak", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": sorted(r["ms"] for r in reps)[len(reps) // 2], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "c3b: papers100M-shaped history layer batched to 20 M edges, %d measurements with "
                                   "freshly allocated tensors" % len(reps)},
            "min_frac": fr[0], "max_frac": fr[-1], "measurements": reps}


def run_copy(args):
    """Plain device copy of known size: the calibration point for the HBM traffic counters."""
    import torch
    n = 1 << 30  # 4 GiB of fp32 read, 4 GiB written
    x = torch.ones(n, device="cuda:0")
    y = torch.empty_like(x)
    sec = timed_steps(lambda: y.copy_(x), args.steps, args.warmup)
    return {"metric": "copy GB/s (read+write)", "value": 2 * n * 4 / sec / 1e9, "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True,
            "config": {"workload": "copy: 4 GiB fp32 device-to-device copy (4 GiB read + 4 GiB written)"}}


def device_power_law_graph(N, mean_degree, dev, gen, max_degree=100_000):
    """CSR of a directed graph generated on the device: log-normal out-degrees (sigma 1.2) with the
    given mean, neighbour ids skewed towards popular nodes (u^3 over the id range, scattered by a
    multiplicative hash).  Multi-edges are possible, as in raw edge lists."""
    import math

    import torch
    sigma = 1.2
    mu = math.log(mean_degree) - sigma * sigma / 2
    deg = torch.exp(mu + sigma * torch.randn(N, device=dev, generator=gen)).floor_().clamp_(0, max_degree).long()
    indptr = torch.zeros(N + 1, dtype=torch.int64, device=dev)
    torch.cumsum(deg, 0, out=indptr[1:])
    del deg
    E = int(indptr[-1])
    indices = torch.empty(E, dtype=torch.int64, device=dev)
    chunk = 100_000_000
    for lo in range(0, E, chunk):
        hi = min(E, lo + chunk)
        u = torch.rand(hi - lo, device=dev, generator=gen, dtype=torch.float64)
        v = (u * u * u * N).long().clamp_(0, N - 1)
        indices[lo:hi] = (v * 2654435761) % N
        del u, v
    return indptr, indices


def run_dispatch(args):
    """What a zero-copy host read costs the kernels that run beside it: a HIP graph of 60 one-element kernels
    (nothing but their dispatch) replayed alone, beside a gather of 90 000 rows from pinned host memory on a stream
    kept to 16 compute units, and beside the same gather from device memory on the same stream."""
    import torch

    import hiscache_backend as be

    dev = "cuda:0"
    N, F, n_rows, n_kernels = 4_000_000, 128, 90_000, 60
    x = torch.zeros(1, device=dev)
    capture = torch.cuda.Stream()
    with torch.cuda.stream(capture):
        for _ in range(3):
            x.add_(1.0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=capture):
        for _ in range(n_kernels):
            x.add_(1.0)
    # the same number of kernels that each move 16 MB inside device memory
    a16 = torch.randn(1 << 22, device=dev)
    b16 = torch.empty_like(a16)
    with torch.cuda.stream(capture):
        b16.copy_(a16)
    torch.cuda.synchronize()
    graph_copy = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph_copy, stream=capture):
        for _ in range(n_kernels):
            b16.copy_(a16)
    host = torch.empty((N, F), dtype=torch.float32, pin_memory=True)
    host.normal_()
    hbm = torch.randn((N, F), device=dev)
    side = be.cu_limited_stream(args.prefetch_cus, torch.device(dev))
    compute = torch.cuda.Stream()
    gen = torch.Generator(device=dev).manual_seed(1)

    def replay_us(beside, g=None):
        g = g or graph
        ids = torch.randint(0, N, (n_rows,), device=dev, generator=gen)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        rows = None
        if beside is not None:
            side.wait_stream(torch.cuda.current_stream())
            rows = be.gather_rows(beside, ids, stream=side)
        with torch.cuda.stream(compute):
            e0.record()
            for _ in range(3):
                g.replay()
            e1.record()
        torch.cuda.synchronize()
        del rows
        return e0.elapsed_time(e1) / 3 * 1e3

    def gather_us(matrix):
        ids = torch.randint(0, N, (n_rows,), device=dev, generator=gen)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(side)
        rows = be.gather_rows(matrix, ids, stream=side)
        e1.record(side)
        torch.cuda.synchronize()
        del rows
        return e0.elapsed_time(e1) * 1e3

    reps = max(3, args.steps)
    alone = min(replay_us(None) for _ in range(reps))
    beside_host = min(replay_us(host) for _ in range(reps))
    beside_hbm = min(replay_us(hbm) for _ in range(reps))
    copies = {"alone": min(replay_us(None, graph_copy) for _ in range(reps)),
              "beside_host_gather": min(replay_us(host, graph_copy) for _ in range(reps)),
              "beside_device_memory_gather": min(replay_us(hbm, graph_copy) for _ in range(reps))}
    return {
        "metric": "us per replay of a 60-kernel graph", "value": alone, "unit": "us", "n_gpus": 1, "steps": reps,
        "warmup": 0, "ms_per_step": alone * 1e-3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "dispatch: %d one-element kernels in a HIP graph; beside them a gather of %d rows x %d "
                               "fp32 on a stream kept to %d compute units" % (n_kernels, n_rows, F, args.prefetch_cus)},
        "replay_us": {"alone": alone, "beside_host_gather": beside_host, "beside_device_memory_gather": beside_hbm},
        "us_per_kernel": {"alone": alone / n_kernels, "beside_host_gather": beside_host / n_kernels,
                          "beside_device_memory_gather": beside_hbm / n_kernels},
        "replay_us_of_60_copies_of_16MB": copies,
        "gather_us": {"host": gather_us(host), "device_memory": gather_us(hbm)},
    }


def run_trainer(args):
    """Epochs of ``hiscache.HistoryTrainer`` over a dataset directory of the plumbing configuration's shape
    (100 k nodes, degree 15, 128-dim fp32 features, 2-layer SAGE hidden 128, fanout [10, 5], batches of 1000 seeds,
    the reference's flat ``HistoryCache`` with a 15 MB buffer): ms per iteration of the epochs behind the first.
    --recorded, --prefetch (the read-ahead), --hot-fraction, --features-in-hbm and --sampler-replay choose the loop."""
    import tempfile

    import numpy as np
    import torch

    from hiscache import HistoryTrainer, make_config, write_processed

    rng = np.random.default_rng(1)
    N, Fin, H, C, L, deg, n_train, batch = 100_000, 128, 128, 10, 2, 15, 60_000, 1000
    indptr = np.arange(0, (N + 1) * deg, deg, dtype=np.int64)
    indices = rng.integers(0, N, size=N * deg).astype(np.int64)
    feats = rng.standard_normal((N, Fin)).astype(np.float32)
    labels = feats[:, :C].argmax(1).astype(np.int64)              # a node's own features decide its label
    perm = rng.permutation(N)
    epochs = max(2, min(args.steps, 6))
    with tempfile.TemporaryDirectory() as root:
        write_processed(root, indptr, indices, feats, hot_ids=np.argsort(np.bincount(indices, minlength=N), kind="stable"),
                        labels=labels, train_idx=perm[:n_train], valid_idx=perm[n_train:n_train + 10_000])
        cfg = make_config(Fin, C, H, L, method="grad", rate=0.5, staleness_thres=200, device="cuda:0", path=root)
        trainer = HistoryTrainer(cfg, fanout=[10, 5], batch_size=batch, lr=1e-3, num_epochs=epochs, eval_begin=epochs - 1,
                                 cache_bytes=30_000 * Fin * 4, recorded=args.recorded, read_ahead=args.prefetch,
                                 hot_rows=int(N * args.hot_fraction), features_in_device_memory=args.features_in_hbm,
                                 replay_slots=max(args.sampler_replay, 4) if args.sampler_replay else 0)
        trainer.train()
        iters = n_train // batch
        per_epoch = [1e3 * s / iters for s in trainer.epoch_seconds]
        ms = float(np.mean(per_epoch[1:]))
        rec = trainer._step
        res = {
            "metric": "trainer iteration ms (1 GPU)", "value": ms, "unit": "ms", "n_gpus": 1, "steps": iters * (epochs - 1),
            "warmup": iters, "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": "HistoryTrainer on a dataset directory: %d nodes, degree %d, %d-dim fp32 features, "
                                   "2-layer SAGE hidden %d, fanout [10,5], %d batches of %d seeds per epoch, flat "
                                   "HistoryCache of %d rows" % (N, deg, Fin, H, iters, batch, 30_000)},
            "ms_per_iteration_by_epoch": per_epoch, "val_metric": trainer.val_metrics,
            "loop": {"recorded": bool(args.recorded), "read_ahead": bool(trainer.read_ahead),
                     "hot_rows": int(N * args.hot_fraction), "features_in_device_memory": bool(args.features_in_hbm),
                     "sampler_replay_slots": trainer.sampler.replay_slots},
            "recorded": None if rec is None else {"replays": rec.replays, "unrecorded": rec.unrecorded},
        }
        trainer.close()
    return res


def run_sample(args):
    """Layered neighbour sampling on a papers100M-sized graph resident in HBM: time per batch when
    the caller waits for it, and what is left on the training thread when the next batch is
    sampled on the side stream while the current one trains."""
    import numpy as np
    import torch

    from hiscache import NeighborSampler

    dev = "cuda:0"
    s = args.scale
    N = int(111_000_000 * s)
    fanout, n_seed = [15, 10, 5], 1000
    gen = torch.Generator(device=dev).manual_seed(6)
    indptr, indices = device_power_law_graph(N, 14.5, dev, gen)
    E_graph = indices.numel()
    sampler = NeighborSampler(indptr, indices, fanout, seed=6, device=dev, validate=False)
    seed_sets = [torch.randperm(N, device=dev, generator=gen)[:n_seed].contiguous() for _ in range(16)]
    clock = KernelClock()
    shapes = []

    def step(i):
        b = clock(lambda: sampler.sample(seed_sets[i % len(seed_sets)]))
        return b

    for i in range(args.warmup):
        step(i)
    sync()
    clock.reset()
    t0 = time.perf_counter()
    for i in range(args.steps):
        b = step(i)
        shapes.append(list(b.num_node_in_layer.tolist()) + [b.idx.numel()])
    sync()
    sec = (time.perf_counter() - t0) / args.steps
    # prefetched: batch i+1 is launched before batch i is consumed; the consumer does 1 ms of other work
    filler = torch.empty(64 << 20, dtype=torch.float32, device=dev)
    pending = sampler.sample_async(seed_sets[0])
    waits = []
    for i in range(args.steps):
        nxt = sampler.sample_async(seed_sets[(i + 1) % len(seed_sets)])
        for _ in range(4):
            filler.add_(1.0)                       # stands for the training iteration
        torch.cuda.current_stream().synchronize()
        t1 = time.perf_counter()
        pending.get()
        waits.append(time.perf_counter() - t1)
        pending = nxt
    pending.get()
    sync()
    # host time of one sample_async (the view emitted with the batch), launched kernel by kernel and replayed
    # from the slots' HIP graphs; the device is idle when each call starts
    host_us, latency_ms = {}, {}
    del sampler
    for name, slots in (("launched", 0), ("replayed", 4)):
        sm = NeighborSampler(indptr, indices, fanout, seed=6, device=dev, validate=False, emit_view=True,
                             replay_slots=slots)
        t_host = t_done = 0.0
        n_rep = max(args.steps, 20)
        for i in range(8 + n_rep):
            sync()
            t0 = time.perf_counter()
            p = sm.sample_async(seed_sets[i % len(seed_sets)])
            t1 = time.perf_counter()
            sync()
            t2 = time.perf_counter()
            p.get()
            if i >= 8:
                t_host += t1 - t0
                t_done += t2 - t0
        host_us[name], latency_ms[name] = 1e6 * t_host / n_rep, 1e3 * t_done / n_rep
        del sm
    mean = np.mean(np.asarray(shapes, dtype=np.float64), axis=0)
    edges = float(mean[-1])
    return {
        "metric": "sampled edges per second (1 GPU, layered neighbour sampling)", "value": edges / sec,
        "unit": "edges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int64", "data": "synthetic",
        "config": {"workload": "sample: graph of %d nodes / %d edges in HBM, fanout %s, %d seeds; mean batch nodes "
                               "%s, edges %d" % (N, E_graph, fanout, n_seed, [int(x) for x in mean[:-1]], int(edges))},
        "device_ms_per_batch": clock.mean_ms(),
        "wait_ms_when_prefetched": float(np.mean(waits) * 1e3),
        "with_view_host_us_per_batch": host_us,
        "with_view_ms_until_batch_is_ready": latency_ms,
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the reference's multi-GPU trainer "
              "and comm.cu are out of scope); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    import hiscache_backend as be
    be.load_library()
    if args.workload in ("c2", "c2row"):
        res, shape = run_c2(args, row_mode=(args.workload == "c2row"))
        torch.cuda.empty_cache()
        if args.workload == "c2" and not args.headline_only:
            # the two other kernel figures of the path, in the same line: the fused admission microbenchmark
            # and the papers100M-shaped history layer batched to 20 M edges
            c4 = run_c4(args)
            torch.cuda.empty_cache()
            res["kernels"]["c4"] = {"workload": c4["config"]["workload"], "ms": c4["ms_per_step"],
                                    "rows_per_s": c4["value"],
                                    "algorithmic_bytes": c4["roofline"]["algorithmic_bytes"],
                                    "GBps": c4["roofline"]["achieved"], "frac": c4["roofline"]["frac"],
                                    "traffic": c4["roofline"]["traffic"]}
            c3b = c3_batched_layer(args)["detail"]
            torch.cuda.empty_cache()
            res["kernels"]["c3_batched"] = c3b
            # the other half of the metric, per-iteration ms at one GPU: the papers100M- and mag240M-shaped
            # training iterations at their real batch shapes (a fresh batch every iteration)
            it_args = argparse.Namespace(**vars(args))
            it_args.steps, it_args.warmup = ITERATION_STEPS, ITERATION_WARMUP
            res["iterations"] = {}
            # c3_sampled: the same iteration fed by the device sampler from a papers100M-sized graph in HBM
            # (batches of about 236 k edges), features read one batch ahead on a CU-limited stream
            sm_args = argparse.Namespace(**vars(it_args))
            sm_args.with_sampler, sm_args.prefetch = True, True
            # c3_sampled_features_in_hbm: a variant beside the configuration's own placement -- the feature matrix
            # in device memory next to the table (288 GB hold both for papers100M), no read-ahead needed
            hb_args = argparse.Namespace(**vars(it_args))
            hb_args.with_sampler, hb_args.features_in_hbm = True, True
            # c3: the features of the next batch are read ahead on the CU-limited stream (it pays since the loop
            # became bound by the GPU; the mag240M-shaped loop is bound by the host and goes without)
            c3_args = argparse.Namespace(**vars(it_args))
            c3_args.prefetch = True
            # *_recorded: the same loops with the iteration recorded once per padded batch shape in a HIP graph
            # and replayed (hiscache.RecordedIteration): one staging launch and one replay per batch
            r1_args = argparse.Namespace(**vars(it_args))
            r1_args.recorded, r1_args.no_cpu_baseline = True, True
            r3_args = argparse.Namespace(**vars(c3_args))
            r3_args.recorded = True
            rh_args = argparse.Namespace(**vars(hb_args))
            rh_args.recorded = True
            # c3_features_in_hbm(_recorded): the configuration's own batches with the feature matrix in device memory
            # beside the table (57 + 57 GB for papers100M: what 288 GB are for) -- no host link in the iteration
            fh_args = argparse.Namespace(**vars(it_args))
            fh_args.features_in_hbm = True
            fr_args = argparse.Namespace(**vars(fh_args))
            fr_args.recorded = True
            r5_args = argparse.Namespace(**vars(it_args))
            r5_args.recorded, r5_args.prefetch = True, True      # once replayed, this loop too gains from the read-ahead
            # c3_sampled_hot_rows: between the two placements -- the matrix in host memory, copies of the rows of the
            # 30% of the nodes with the most incoming edges in device memory (17 GB); the others are read ahead
            ht_args = argparse.Namespace(**vars(sm_args))
            ht_args.hot_fraction = 0.3
            rt_args = argparse.Namespace(**vars(ht_args))
            rt_args.recorded = True
            runs = (("c1", it_args, lambda: run_c1(it_args)),
                    ("c1_recorded", r1_args, lambda: run_c1(r1_args)),
                    ("c3", c3_args, lambda: run_c3(c3_args, with_batched=False)),
                    ("c3_recorded", r3_args, lambda: run_c3(r3_args, with_batched=False)),
                    ("c3_features_in_hbm", fh_args, lambda: run_c3(fh_args, with_batched=False)),
                    ("c3_features_in_hbm_recorded", fr_args, lambda: run_c3(fr_args, with_batched=False)),
                    ("c5", it_args, lambda: run_c5(it_args)),
                    ("c5_recorded", r5_args, lambda: run_c5(r5_args)),
                    ("c3_sampled", sm_args, lambda: run_c3(sm_args, with_batched=False)),
                    ("c3_sampled_hot_rows", ht_args, lambda: run_c3(ht_args, with_batched=False)),
                    ("c3_sampled_hot_rows_recorded", rt_args, lambda: run_c3(rt_args, with_batched=False)),
                    ("c3_sampled_features_in_hbm", hb_args, lambda: run_c3(hb_args, with_batched=False)),
                    ("c3_sampled_features_in_hbm_recorded", rh_args, lambda: run_c3(rh_args, with_batched=False)))
            for name, used_args, fn in runs:
                gc.collect()
                torch.cuda.empty_cache()
                r = fn()
                res["iterations"][name] = {
                    "workload": r["config"]["workload"], "ms": r["ms_per_step"], "steps": r["steps"],
                    "warmup": r["warmup"], "transposed_view": r["transposed_view"],
                    "feature_read_ahead": bool(used_args.prefetch),
                    "ms_per_chunk_of_steps": r.get("ms_per_chunk_of_steps"),
                    "phases_ms": r["phases_ms"], "phases_host_enqueue_ms": r["phases_host_enqueue_ms"]}
                if r.get("feature_rows_in_device_memory"):
                    res["iterations"][name]["feature_rows"] = {
                        "needed_last_batch": r["feature_rows_read_last_batch"],
                        "over_host_link_last_read": r["feature_rows_over_host_link_last_read"],
                        "copies_in_device_memory": r["feature_rows_in_device_memory"]}
                if r.get("recorded"):            # the whole iteration is the one phase called "load"
                    res["iterations"][name]["recorded"] = r["recorded"]
                if "cpu_baseline" in r:          # c1, the CPU-runnable configuration: the same iteration on the host
                    res["iterations"][name]["cpu_ms"] = r["cpu_baseline"]["value"]
                    res["iterations"][name]["cpu_cores"] = r["cpu_baseline"]["cores"]
            gc.collect()
            torch.cuda.empty_cache()
        if not args.no_cpu_baseline:
            res["cpu_baseline"] = cpu_baseline_c2(shape)
    elif args.workload == "c2w":
        res = run_c2w(args)
    elif args.workload == "c4":
        res = run_c4(args)
        if not args.no_cpu_baseline:
            res["cpu_baseline"] = cpu_baseline_c4(int(2_000_000 * args.scale), 256)
    elif args.workload == "layer":
        res = run_layer(args)
    elif args.workload == "c3b":
        res = run_c3b(args)
    elif args.workload == "copy":
        res = run_copy(args)
    elif args.workload == "c5":
        res = run_c5(args)
    elif args.workload == "c1":
        res = run_c1(args)
    elif args.workload == "sample":
        res = run_sample(args)
    elif args.workload == "trainer":
        res = run_trainer(args)
    elif args.workload == "dispatch":
        res = run_dispatch(args)
    else:
        res = run_c3(args)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
