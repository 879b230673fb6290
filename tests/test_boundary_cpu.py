"""The C-ABI library loads without a GPU, exports every symbol the header declares, and its
argument checks return status codes (no kernel is launched here)."""
import ctypes
import os
import re
import types

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hiscache_hip.h")


def header_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hc_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_agree():
    import hiscache_backend as be
    assert header_functions() == be.exported_symbols()


def test_library_exports_every_declared_symbol():
    import hiscache_backend as be
    lib = be.load_library()
    for name in header_functions():
        assert hasattr(lib, name), name
    assert b"gfx950" in lib.hc_version()
    assert lib.hc_strerror(0) == b"ok"
    assert lib.hc_device_count() >= 0


def test_argument_errors_are_status_codes():
    import hiscache_backend as be
    lib = be.load_library()
    null = ctypes.c_void_p(None)
    # negative row count, zero feature width
    assert lib.hc_aggr_fwd(0, null, null, null, 0, null, null, 0, 0, null, 1, null, -1, 4, 0, null, 0, null) == 1
    assert lib.hc_aggr_fwd(0, null, null, null, 0, null, null, 0, 0, null, 1, null, 4, 0, 0, null, 0, null) == 1
    # missing pointers
    assert lib.hc_aggr_fwd(0, null, null, null, 0, null, null, 0, 0, null, 1, null, 4, 4, 4, null, 0, null) == 1
    buf = np.zeros(64, np.int64)
    p = ctypes.c_void_p(buf.ctypes.data)
    # unknown dtype / substitution mode
    assert lib.hc_aggr_fwd(0, p, p, p, 7, null, null, 0, 0, null, 1, p, 4, 4, 4, null, 0, null) == 2
    assert lib.hc_aggr_fwd(9, p, p, p, 0, null, null, 0, 0, null, 1, p, 4, 4, 4, null, 0, null) == 1
    # heads need edge values; history map needs a buffer
    assert lib.hc_aggr_fwd(0, p, p, p, 0, null, null, 0, 0, null, 2, p, 4, 4, 4, null, 0, null) == 1
    assert lib.hc_aggr_fwd(0, p, p, p, 0, p, null, 0, 4, null, 1, p, 4, 4, 4, null, 0, null) == 1
    # grad_check: bad enums, missing workspace
    args = [p, null, p, p, null, null, p, p, 0, 0, 0, p, null, null, p, 0, 8, p, p, null, p, 0, 4, 4]
    assert lib.hc_grad_check(*args, null, 0, null) == 4
    bad = list(args); bad[9] = 5
    assert lib.hc_grad_check(*bad, p, 512, null) == 1
    bad = list(args); bad[15] = 9
    assert lib.hc_grad_check(*bad, p, 512, null) == 2
    tiles = 2_000_000 // 64              # one count byte per 64-row tile, one 8-byte prefix per 32 tiles
    assert tiles + 8 * (tiles // 32) <= lib.hc_grad_check_workspace_bytes(2_000_000) <= 2 * tiles
    assert lib.hc_row_scores(null, null, 4, 4, 0, null) == 1
    assert lib.hc_gather_rows(p, 5, 4, p, null, p, 0, 0, 2, 4, null) == 2
    assert lib.hc_gather_rows(p, 0, 4, p, null, p, 9, 0, 2, 4, null) == 2
    assert lib.hc_count_history(null, null, null, 0, null, 4, 4, 1, 2, null) == 1
    # the batch's shared view: missing pointers, capacities beyond the device-sized build, missing workspace,
    # widths off the relational kernel's list -- all refused before anything is launched
    assert lib.hc_aggr_bwd_batch_view(null, null, null, null, null, null, null, 0, 0, 4, 64, 4, null, 0, null) == 1
    assert lib.hc_aggr_bwd_batch_view(p, p, p, p, null, p, p, 64, 8, 4, 64, 4, null, 0, null) == 1   # hbuf without map
    big = (1 << 24) + 1
    assert lib.hc_transpose_dev_workspace_bytes(big, 10) == 0 and lib.hc_transpose_dev_workspace_bytes(10, big) == 0
    need = lib.hc_transpose_dev_workspace_bytes(1000, 100)
    assert need >= 4 * 4 * 1000 + 4 * 101
    assert lib.hc_build_transpose_dev(p, p, p, p, p, big, 10, p, p, null, null, p, 1 << 40, null) == 5
    assert lib.hc_build_transpose_dev(p, p, p, p, p, 1000, 100, p, p, null, null, null, 0, null) == 4
    assert lib.hc_build_transpose_dev(p, p, null, p, p, 1000, 100, p, p, null, null, p, need, null) == 1
    assert lib.hc_build_transpose_dev_deg(p, p, p, p, p, 1000, 100, p, p, null, null, null, null, 0, null) == 4
    assert lib.hc_aggr_bwd_batch_view_typed(p, p, p, p, p, 8, 3, null, p, p, 4, 100, 4, null) == 5
    assert lib.hc_aggr_bwd_batch_view_typed(p, p, p, p, null, 8, 3, null, p, p, 4, 64, 4, null) == 1
    assert lib.hc_aggr_bwd_batch_view_typed(p, p, p, p, p, 8, 0, null, p, p, 4, 64, 4, null) == 1
    assert lib.hc_fixup_rows(p, 0, 4, p, p, null, p, 0, 2, 4, null) == 1       # the guessed mask is missing
    assert lib.hc_fixup_rows(p, 7, 4, p, p, p, p, 0, 2, 4, null) == 2
    assert lib.hc_stream_create_cu_limited(0, p) == 1 and lib.hc_stream_create_cu_limited(8, null) == 1
    assert lib.hc_stream_destroy(null) == 0
    for code in range(0, 8):
        assert lib.hc_strerror(code)


def test_python_shim_refuses_cpu_tensors():
    import torch
    import hiscache_backend as be
    x = torch.zeros(4, 4)
    ptr = torch.zeros(5, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="GPU"):
        be.aggr_forward_history(x, ptr, ptr, torch.tensor([]), torch.tensor([]), 0, 4)
    with pytest.raises(RuntimeError, match="GPU"):
        be.count_history_reconstruct(ptr, ptr, ptr, 4, 1, 2)
    with pytest.raises(RuntimeError):
        be.gather_rows(torch.zeros(4, 4), ptr)          # neither on the GPU nor pinned


def test_config_and_synthetic_batch_layout():
    from hiscache import make_config
    from hiscache.synthetic import direct_power_law_batch, sample_layered_batch, uniform_graph, zipf_degrees
    cfg = make_config(128, 10, 128, 2)
    assert cfg.dl.dataset.feature_dim == cfg["dl"]["dataset"]["feature_dim"] == 128
    assert cfg.history.get("store_last_layer", False) is False
    rng = np.random.default_rng(0)
    indptr, indices = uniform_graph(2000, 15, 1)
    s = sample_layered_batch(indptr, indices, rng.choice(2000, 50, replace=False), [10, 5], rng)
    nnl = s["num_node_in_layer"]
    assert len(s["ptr"]) - 1 == nnl[1] and nnl[0] == 50 and nnl[2] == len(s["sub_to_full"])
    assert len(np.unique(s["sub_to_full"])) == len(s["sub_to_full"])
    assert s["idx"][: s["ptr"][nnl[0]]].max() < nnl[1]             # seeds' neighbours are within 1 hop
    for r in range(len(s["ptr"]) - 1):                              # sampled edges exist in the graph
        full = s["sub_to_full"][r]
        nb = s["sub_to_full"][s["idx"][s["ptr"][r]:s["ptr"][r + 1]]]
        assert np.isin(nb, indices[indptr[full]:indptr[full + 1]]).all()
    d = direct_power_law_batch(10**7, 100, [15, 10, 5], 2.0, 3)
    nnl = d["num_node_in_layer"]
    assert len(d["ptr"]) - 1 == nnl[2] and d["idx"].max() < nnl[3]
    assert len(np.unique(d["sub_to_full"])) == len(d["sub_to_full"])
    deg = zipf_degrees(10000, 200000, 2.1, 5000, rng)
    assert deg.sum() == 200000 and deg.min() >= 1 and deg.max() <= 5000


def test_processed_dataset_files_round_trip(tmp_path):
    """The on-disk layout of /root/reference/hiscache/history_cache.py:17-20,124-142 and
    test/test_cache.py:19-56: raw int64 / float arrays plus num_nodes.txt."""
    from hiscache import ProcessedDataset, write_processed
    from hiscache.synthetic import uniform_graph
    rng = np.random.default_rng(5)
    indptr, indices = uniform_graph(200, 6, 5)
    feats = rng.standard_normal((200, 12)).astype(np.float16)
    hot = rng.permutation(200)
    labels = rng.integers(0, 4, size=200)
    train = rng.choice(200, size=50, replace=False)
    d = write_processed(tmp_path, indptr, indices, feats, hot, labels, train)
    assert open(os.path.join(d, "num_nodes.txt")).read().strip() == "200"
    assert os.path.getsize(os.path.join(d, "node_features.dat")) == 200 * 12 * 2
    ds = ProcessedDataset(tmp_path, 12, np.float16)
    assert ds.num_nodes == 200
    p, i = ds.graph()
    np.testing.assert_array_equal(p, indptr)
    np.testing.assert_array_equal(i, indices)
    np.testing.assert_array_equal(ds.hot_ids(), hot)
    np.testing.assert_array_equal(ds.labels(), labels)
    np.testing.assert_array_equal(ds.train_idx(), train)
    np.testing.assert_array_equal(np.fromfile(os.path.join(d, "sorted_indices.dat"), dtype=np.int64), hot)
    # a truncated CSR file is refused
    np.asarray(indices[:-3], np.int64).tofile(os.path.join(d, "csr_idx_undirected.dat"))
    with pytest.raises(ValueError):
        ds.graph()


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert p.returncode == 2 and "one GPU" in p.stderr and p.stdout.strip() == ""


def test_header_is_plain_c_and_links(tmp_path):
    """include/hiscache_hip.h compiles as C11 and a C program linked against the library can call it
    (no GPU is touched: hc_version / hc_strerror / hc_device_count only)."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib_dir = os.path.join(root, "history-cache_amd")
    if not os.path.exists(os.path.join(lib_dir, "libhiscache_hip.so")):
        pytest.skip("library not built")
    src = tmp_path / "abi_check.c"
    src.write_text('#include <stdio.h>\n#include "hiscache_hip.h"\n'
                   'int main(void) { printf("%s|%s|%d\\n", hc_version(), hc_strerror(HC_EWORKSPACE), '
                   'hc_device_count() >= 0); return 0; }\n')
    exe = tmp_path / "abi_check"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                    str(src), "-o", str(exe), "-L", lib_dir, "-lhiscache_hip", "-Wl,-rpath," + lib_dir],
                   check=True, capture_output=True, text=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, timeout=60).stdout
    assert out.startswith("hiscache_hip") and out.strip().endswith("|1")


def test_relational_gemm_spellings_equal_the_single_gemm():
    """The split spellings of the relational layer's two large GEMMs (over relations forward, over row
    slabs for the weight gradient) against the plain products, on both sides of the size switch and with
    row counts that leave a remainder."""
    import torch
    from hiscache import history_model as hm
    torch.manual_seed(0)
    for n, K, Fin, H in ((37, 5, 16, 8), (101, 5, 512, 24), (8, 3, 700, 4), (7, 5, 512, 6), (64, 1, 4096, 8)):
        agg = torch.randn(n, K, Fin, dtype=torch.float64)
        w = torch.randn(K, Fin, H, dtype=torch.float64)
        g = torch.randn(n, H, dtype=torch.float64)
        want = agg.reshape(n, K * Fin) @ w.reshape(K * Fin, H)
        assert torch.allclose(hm._rel_matmul(agg, w), want, rtol=1e-12, atol=1e-12)
        want_g = (agg.reshape(n, K * Fin).t() @ g).view(K, Fin, H)
        got_g = hm._rel_weight_grad(agg, g)
        assert got_g.shape == (K, Fin, H) and torch.allclose(got_g, want_g, rtol=1e-12, atol=1e-12)


def test_weight_gradient_slab_spelling_equals_the_single_gemm():
    import torch
    from hiscache import history_model as hm
    torch.manual_seed(3)
    for n in (5, 8191, 8192, 9000, 20_001):
        g = torch.randn(n, 12, dtype=torch.float64)
        x = torch.randn(n, 20, dtype=torch.float64)
        assert torch.allclose(hm._weight_grad(g, x), g.t() @ x, rtol=1e-11, atol=1e-9)
    x_view = torch.randn(9000, 40, dtype=torch.float64)[:, :20]      # rows of a wider matrix
    g = torch.randn(9000, 12, dtype=torch.float64)
    assert torch.allclose(hm._weight_grad(g, x_view), g.t() @ x_view, rtol=1e-11, atol=1e-9)


def test_bn_relu_takes_the_torch_operators_off_the_gpu():
    """Without a GPU tensor (or in evaluation mode) bn_relu is exactly relu(bn(x + bias)), module state
    included."""
    import torch
    import torch.nn.functional as F
    from hiscache.history_model import bn_relu
    torch.manual_seed(1)
    a, b = torch.nn.BatchNorm1d(12), torch.nn.BatchNorm1d(12)
    b.load_state_dict(a.state_dict())
    x, bias = torch.randn(9, 12), torch.randn(12)
    for mode in ("train", "eval"):
        getattr(a, mode)(), getattr(b, mode)()
        assert torch.equal(bn_relu(x, a, bias), F.relu(b(x + bias)))
        assert torch.equal(a.running_mean, b.running_mean) and torch.equal(a.running_var, b.running_var)
        assert int(a.num_batches_tracked) == int(b.num_batches_tracked)


def test_batched_history_layer_block_layout():
    """Rows, edge offsets and source shifts of the block the benchmark and the full-size test build."""
    from hiscache.synthetic import batched_history_layer, direct_power_law_batch
    samples = [direct_power_law_batch(1_000_000, 50, [5, 4, 3], 2.0, 3 + i, degree_scale=2.0) for i in range(3)]
    ptr, idx, R, E, N = batched_history_layer(samples, 4000)
    assert ptr[0] == 0 and ptr[-1] == E == len(idx) and len(ptr) == R + 1 and E >= 4000
    assert (np.diff(ptr) >= 0).all() and idx.min() >= 0 and idx.max() < N
    row0, col0, k = 0, 0, 0
    while row0 < R:
        smp = samples[k % 3]
        n1, n2 = int(smp["num_node_in_layer"][1]), int(smp["num_node_in_layer"][2])
        e0, e1 = int(ptr[row0]), int(ptr[row0 + n1])
        np.testing.assert_array_equal(ptr[row0:row0 + n1 + 1] - e0, smp["ptr"][: n1 + 1])
        np.testing.assert_array_equal(idx[e0:e1] - col0, smp["idx"][: e1 - e0])
        row0, col0, k = row0 + n1, col0 + n2, k + 1
    assert row0 == R and col0 == N


def test_column_sums_by_matrix_vector_product():
    import torch
    from hiscache import history_model as hm
    torch.manual_seed(2)
    for n in (1, 7, 1024, 1025, 5000):
        g = torch.randn(n, 9, dtype=torch.float64)
        assert torch.allclose(hm._column_sums(g), g.sum(0), rtol=1e-12, atol=1e-12)


def test_cu_limited_stream_teardown_is_idempotent(monkeypatch):
    """The exit hook that gives CU-limited streams back destroys every handle once, drops the per-stream
    scratch kept for it, survives a device that can no longer synchronise, and does nothing the second time;
    releasing a stream by hand takes it off the hook's list."""
    import hiscache_backend as be

    destroyed = []

    class Lib:
        def hc_stream_destroy(self, handle):
            destroyed.append(handle.value)
            return 0

    def no_device():
        raise RuntimeError("no device")

    monkeypatch.setattr(be, "load_library", lambda: Lib())
    monkeypatch.setattr(be.torch.cuda, "synchronize", no_device)
    monkeypatch.setattr(be, "_cu_stream_handles", [0x1000, 0x2000, 0x3000])
    monkeypatch.setattr(be, "_ws_cache", {(0, 0x1000): "a", (0, 0x2000): "b", (0, 0): "default"})
    monkeypatch.setattr(be, "_tickets", {(0, 0x2000): "t"})

    class Stream:
        cuda_stream = 0x2000
        waited = 0

        def synchronize(self):
            Stream.waited += 1

    assert be.release_cu_limited_stream(Stream()) is True
    assert Stream.waited == 1 and destroyed == [0x2000]
    assert be.release_cu_limited_stream(Stream()) is False          # already gone
    assert (0, 0x2000) not in be._ws_cache and (0, 0x2000) not in be._tickets
    be._destroy_cu_streams()
    assert sorted(destroyed) == [0x1000, 0x2000, 0x3000] and be._cu_stream_handles == []
    assert be._ws_cache == {(0, 0): "default"}
    be._destroy_cu_streams()
    assert len(destroyed) == 3


def test_recorded_iteration_shape_family():
    """The padded shapes of hiscache.RecordedIteration: the smallest member of the family that holds the batch,
    rows rounded up, a layer's rows a prefix of the next layer's; another number of seeds is not in the family."""
    from types import SimpleNamespace

    import torch

    from hiscache import RecordedIteration
    rec = RecordedIteration(None, SimpleNamespace(device=torch.device("cpu")), None, 3, step=1.125, round_to=256)
    base = [1000, 5800, 25_800, 89_000]
    assert rec._key_for(base, 88_000) == 0
    caps, e_cap = rec._shape(0)
    assert caps == [1000, 5888, 25_856, 89_088] and e_cap == 88_064
    rng = np.random.default_rng(0)
    for _ in range(300):
        f = rng.uniform(0.6, 1.6, size=4)
        nnl = [1000] + sorted(int(b * x) for b, x in zip(base[1:], f[:3]))
        n_e = int(88_000 * f[3])
        j = rec._key_for(nnl, n_e)
        caps, e_cap = rec._shape(j)
        assert all(a <= c for a, c in zip(nnl, caps)) and n_e <= e_cap
        assert caps == sorted(caps)
        assert not rec._holds(j - 1, nnl, n_e)                       # the smallest one
    assert rec._key_for([999] + base[1:], 88_000) is None
    # a hop that adds no node: the caps stay ordered
    rec2 = RecordedIteration(None, SimpleNamespace(device=torch.device("cpu")), None, 2, round_to=64)
    caps, e_cap = rec2._shape(rec2._key_for([500, 500, 500], 0))
    assert caps[0] == 500 and caps == sorted(caps) and all(c >= 500 for c in caps) and e_cap >= 0


def test_trainer_hands_out_every_batch_once_and_reads_one_batch_ahead():
    """The trainer's batch pipeline with stand-ins for the sampler and the recorded step (no GPU): every chunk of the
    split becomes one batch, in order; a batch is sampled while the one before is in use; with the read-ahead the
    feature read of batch k + 1 is started before batch k is handed out, and never for a batch twice."""
    import torch
    from hiscache.history_trainer import HistoryTrainer, _option
    from hiscache import make_config

    events = []

    class Pending:
        def __init__(self, seeds):
            self.seeds = seeds

        def get(self):
            events.append(("got", int(self.seeds[0])))
            return types.SimpleNamespace(seeds=self.seeds)

    class Sampler:
        def sample_async(self, seeds):
            events.append(("sampling", int(seeds[0])))
            return Pending(seeds)

    class Step:
        def prefetch(self, batch):
            events.append(("read", int(batch.seeds[0])))

    for n_ids, batch_size in ((10, 4), (4, 4), (1, 4), (0, 4), (23, 5)):
        for read_ahead in (False, True):
            t = object.__new__(HistoryTrainer)
            t.device, t.batch_size, t.sampler, t._step, t.num_layers = torch.device("cpu"), batch_size, Sampler(), Step(), 2
            events.clear()
            ids = torch.arange(n_ids) * 10
            firsts = []
            for batch in t._batches(ids, shuffle=False, read_ahead=read_ahead):
                events.append(("train", int(batch.seeds[0])))
                firsts.append(int(batch.seeds[0]))
            want = [int(ids[lo]) for lo in range(0, n_ids, batch_size)]
            assert firsts == want
            assert [e[1] for e in events if e[0] == "sampling"] == want          # every chunk sampled once, in order
            for k, first in enumerate(want):
                at = events.index(("train", first))
                if k + 1 < len(want):                                            # the next batch is under way by then
                    assert events.index(("sampling", want[k + 1])) < at
                    if read_ahead:
                        assert events.index(("read", want[k + 1])) < at
            reads = [e[1] for e in events if e[0] == "read"]
            assert reads == (want[1:] if read_ahead else [])

    cfg = make_config(8, 2, 8, 2)
    assert _option(cfg, "train.model.num_layers", 7) == 2
    assert _option(cfg, "train.train.num_epochs", 7) == 7 and _option(cfg, "dl.sampler.train.batch_size", None) is None
