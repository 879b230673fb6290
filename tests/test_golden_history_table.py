"""Golden vectors produced by the reference's own HistoryTable.lookup / evict_by_both / evict_by_staleness
(tests/golden/gen_history_table_golden.py ran /root/reference/hiscache/history_table.py on CPU tensors; the
admission kernel of that class is CUDA code and did not run: entries were written into the tables directly,
as the tests here write them).  The CPU restatement (oracle.host_model) and the GPU HistoryTable must both
reproduce them: slots, compact ids, gathered rows and the three maps after eviction, exactly."""
import hashlib
import os
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden", "history_table_golden.npz")
sys.path.insert(0, os.path.join(HERE, "golden"))

# sha256 over the sub_to_full arrays of the scenario's batches: the inputs are rebuilt from seeds, and a
# different random stream would otherwise show up as a wall of mismatches
INPUT_DIGEST = {"grad": "5ca335c66116bb126b5e91c48bc45d5c3504eb97ff6655bdf8e56c368589294b", "staleness": "e97045f9c03b730e635b98490e2e38a78355ad031a070583f79070ea6c999e41"}


def load():
    return np.load(GOLD, allow_pickle=False)


def scenario_of(name):
    import gen_history_table_golden as gen       # inputs only; nothing of the reference is read at import
    steps = gen.scenario(name)
    h = hashlib.sha256()
    for s in steps:
        h.update(np.ascontiguousarray(s["batch"]["sub_to_full"]).tobytes())
    assert h.hexdigest() == INPUT_DIGEST[name], "the scenario's inputs are not the ones the fixture was made from"
    return gen, steps


@pytest.mark.parametrize("name", ["grad", "staleness"])
def test_oracle_reproduces_reference_table_vectors(orc, name):
    from oracle import host_model
    g = load()
    gen, steps = scenario_of(name)
    case = gen.CASES[name]
    L = gen.LAYERS - 1
    widths = [gen.FIN, gen.HID]
    f2h = [torch.full((gen.N,), -1, dtype=torch.int64) for _ in range(L)]
    h2f = [torch.full((gen.SLOTS[l],), -1, dtype=torch.int64) for l in range(L)]
    chk = [torch.full((gen.SLOTS[l],), -1, dtype=torch.int64) for l in range(L)]
    buf = [torch.zeros(gen.SLOTS[l], widths[l]) for l in range(L)]
    evicted_by_score = 0
    for it, step in enumerate(steps, start=1):
        pre = f"{name}_it{it}_"
        b = step["batch"]
        nnl = b["num_node_in_layer"]
        s2f = torch.from_numpy(b["sub_to_full"])
        for l in range(L):
            nodes, rows, order = step["inject"][l]
            k = gen.write_entries(f2h[l], h2f[l], chk[l], buf[l], torch.from_numpy(nodes), torch.from_numpy(rows),
                                  torch.from_numpy(order), it)
            assert k == int(g[pre + f"written{l}"])
        for l in range(L):
            n = int(nnl[gen.LAYERS - 1 - l])
            s2h, rows, compact = host_model.table_lookup(f2h[l], buf[l], s2f, n, int(nnl[0]))
            np.testing.assert_array_equal(s2h.numpy(), g[pre + f"sub_to_history{l}"])
            np.testing.assert_array_equal(compact.numpy(), g[pre + f"compact{l}"])
            np.testing.assert_array_equal(rows.numpy(), g[pre + f"rows{l}"])
            if name == "grad":
                score = torch.from_numpy(orc.row_scores(step["grads"][l], orc.NORM_L1))
                live = int((h2f[l] != -1).sum())
                host_model.evict_by_both(chk[l], h2f[l], f2h[l], s2h, score, case["rate"], it, case["staleness"][l])
                evicted_by_score += live - int((h2f[l] != -1).sum())
            else:
                host_model.evict_by_staleness(chk[l], h2f[l], f2h[l], it, case["staleness"][l])
            np.testing.assert_array_equal(f2h[l].numpy(), g[pre + f"full_to_history{l}"])
            np.testing.assert_array_equal(h2f[l].numpy(), g[pre + f"history_to_full{l}"])
            np.testing.assert_array_equal(chk[l].numpy(), g[pre + f"checkin{l}"])
    if name == "grad":
        assert evicted_by_score > 50


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["grad", "staleness"])
def test_gpu_table_reproduces_reference_table_vectors(name):
    from hiscache import HistoryTable, make_config
    dev = "cuda:0"
    g = load()
    gen, steps = scenario_of(name)
    case = gen.CASES[name]
    cfg = make_config(gen.FIN, gen.CLASSES, gen.HID, gen.LAYERS, method=case["method"], rate=case["rate"],
                      staleness_thres=list(case["staleness"]), device=dev, model_type="SAGE",
                      buffer_size=list(gen.SLOTS))
    t = HistoryTable(cfg, total_num_node=gen.N)
    L = t.num_layers
    assert L == gen.LAYERS - 1 and t.history_size_layered == [gen.FIN, gen.HID]
    for l in range(L):
        t.history_buffer_layered[l].zero_()
    T = lambda a: torch.from_numpy(a).to(dev)
    for it, step in enumerate(steps, start=1):
        pre = f"{name}_it{it}_"
        b = step["batch"]
        for l in range(L):
            nodes, rows, order = step["inject"][l]
            k = gen.write_entries(t.full_to_history_layered[l], t.history_to_full_layered[l], t.checkin_iter[l],
                                  t.history_buffer_layered[l], T(nodes), T(rows), T(order), it)
            assert k == int(g[pre + f"written{l}"])
        batch = SimpleNamespace(ptr=T(b["ptr"]), idx=T(b["idx"]), sub_to_full=T(b["sub_to_full"]),
                                num_node_in_layer=torch.from_numpy(b["num_node_in_layer"]),
                                y=torch.zeros(int(b["num_node_in_layer"][0]), dtype=torch.int64, device=dev), x=None)
        t.lookup(batch.sub_to_full, batch.num_node_in_layer)
        t.history_out = []
        for l in range(L):
            np.testing.assert_array_equal(t.sub_to_history[l].cpu().numpy(), g[pre + f"sub_to_history{l}"])
            np.testing.assert_array_equal(t.sub_to_history_layered[l].cpu().numpy(), g[pre + f"compact{l}"])
            np.testing.assert_array_equal(t.tmp_history_buffer_layered[l].detach().cpu().numpy(), g[pre + f"rows{l}"])
            assert t.tmp_history_buffer_layered[l].requires_grad == (name == "grad")
            grad = T(step["grads"][l])
            h = torch.zeros_like(grad).requires_grad_(True)
            h.grad = grad
            t.history_out.append(h)
        t.evict_history(batch, it)
        for l in range(L):
            np.testing.assert_array_equal(t.full_to_history_layered[l].cpu().numpy(), g[pre + f"full_to_history{l}"])
            np.testing.assert_array_equal(t.history_to_full_layered[l].cpu().numpy(), g[pre + f"history_to_full{l}"])
            np.testing.assert_array_equal(t.checkin_iter[l].cpu().numpy(), g[pre + f"checkin{l}"])
