"""Generates tests/golden/history_table_golden.npz by running the reference's own
``HistoryTable.__init__``, ``lookup``, ``evict_by_both`` and ``evict_by_staleness``
(/root/reference/hiscache/history_table.py:11-70, 94-125, 189-251) on CPU tensors.

Run in the build container only (the reference tree is not available elsewhere):

    python tests/golden/gen_history_table_golden.py

The reference module's SOURCE TEXT is read from /root/reference, compiled and executed here (no
importlib loader, no bytecode).  Its two imports that this scenario never calls into are supplied as empty
modules: ``hiscache_backend`` (the CUDA extension: only ``record_history`` and the graph-structure score use
it, neither runs here) and ``hiscache.util`` (a logger).  ``record_history`` is a CUDA kernel and cannot
run; entries enter the tables here by writing the maps directly (slot, owner, check-in iteration, row), the
same writes on both sides of every test, so that ``lookup`` and the two eviction rules see tables in every
state: empty, partly filled, with stale entries, with entries of the batch's own nodes.
Only inputs and outputs are stored; no reference source text is copied.
"""
import logging
import os
import sys
import tempfile
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, os.path.join(ROOT, "history-cache_amd"))  # Config and the synthetic batch generator only
REF = "/root/reference/hiscache/history_table.py"

N, FIN, HID, CLASSES, LAYERS = 20_000, 16, 24, 5, 3
SLOTS = [1500, 1100]
N_ITER = 5
CASES = {"grad": dict(method="grad", rate=0.3, staleness=[2, 3]),
         "staleness": dict(method="staleness", rate=0.3, staleness=[1, 2])}


def load_reference_class():
    saved = {k: sys.modules.get(k) for k in ("hiscache", "hiscache.util", "hiscache.history_table", "hiscache_backend")}
    pkg = types.ModuleType("hiscache")
    pkg.__path__ = []
    util = types.ModuleType("hiscache.util")
    util.log = logging.getLogger("reference")
    sys.modules["hiscache"] = pkg
    sys.modules["hiscache.util"] = util
    sys.modules["hiscache_backend"] = types.ModuleType("hiscache_backend")
    sys.dont_write_bytecode = True
    mod = types.ModuleType("hiscache.history_table")
    mod.__file__ = REF
    mod.__package__ = "hiscache"
    sys.modules["hiscache.history_table"] = mod
    with open(REF, "r", encoding="utf-8") as f:
        code = compile(f.read(), REF, "exec")      # the source text itself, never cached bytecode
    exec(code, mod.__dict__)
    for k, v in saved.items():
        if v is None:
            sys.modules.pop(k, None)
        else:
            sys.modules[k] = v
    return mod.HistoryTable


def table_config(case, root):
    from hiscache.util import make_config
    return make_config(FIN, CLASSES, HID, LAYERS, method=case["method"], rate=case["rate"],
                       staleness_thres=list(case["staleness"]), device="cpu", path=root, model_type="SAGE",
                       buffer_size=list(SLOTS))


def scenario(name):
    """The inputs of case ``name``: batches, the entries written into the tables in front of every
    iteration's lookup, the gradients of the recorded layers.  Rebuilt bit for bit by the tests."""
    from helpers import affine_ids, exact_rows, exact_sum_rows, layered_batch
    seed = {"grad": 31, "staleness": 32}[name]
    rng = np.random.default_rng(seed)
    its = []
    for it in range(1, N_ITER + 1):
        b = layered_batch(rng, N, 60, [6, 5, 4])
        nnl = b["num_node_in_layer"]
        widths = [FIN, HID]
        inject, grads = [], []
        for layer in range(LAYERS - 1):
            n = int(nnl[LAYERS - 1 - layer])
            # half of the new entries belong to nodes of this batch's layer, half to other nodes
            k = 150 + 40 * layer
            own = b["sub_to_full"][:n][rng.permutation(n)[: k // 2]]
            other = affine_ids(N, k - k // 2, 7001 + 10 * it, 17 * it + layer)
            nodes = np.unique(np.concatenate([own, other]))
            rows = exact_rows(seed * 1000 + 10 * it + layer, len(nodes), widths[layer], octaves=3)
            inject.append((nodes, rows, rng.permutation(SLOTS[layer])))
            # gradient rows whose L1 norms are exact however a row is folded
            grads.append(exact_sum_rows(seed * 1000 + 10 * it + layer + 5, n, widths[layer]))
        its.append(dict(batch=b, inject=inject, grads=grads))
    return its


def write_entries(full_to_history, history_to_full, checkin, buffer, nodes, rows, slot_order, it):
    """Entries for the ``nodes`` that have none, in the free slots that come first in ``slot_order``."""
    free = slot_order[history_to_full[slot_order] == -1]
    new = nodes[full_to_history[nodes] == -1][: len(free)]
    slots = free[: len(new)]
    full_to_history[new] = slots
    history_to_full[slots] = new
    checkin[slots] = it
    buffer[slots] = rows[: len(new)]
    return len(new)


def main():
    HistoryTable = load_reference_class()
    out = {"N": N, "Fin": FIN, "H": HID, "layers": LAYERS, "slots": np.asarray(SLOTS), "n_iter": N_ITER}
    with tempfile.TemporaryDirectory() as root:
        os.makedirs(os.path.join(root, "processed"))
        with open(os.path.join(root, "processed", "num_nodes.txt"), "w") as f:
            f.write("%d\n" % N)
        for name, case in CASES.items():
            t = HistoryTable(table_config(case, root))
            assert t.num_layers == LAYERS - 1 and t.history_size_layered == [FIN, HID]
            for layer in range(t.num_layers):
                t.history_buffer_layered[layer].zero_()
            summary = []
            for it, step in enumerate(scenario(name), start=1):
                b = step["batch"]
                pre = f"{name}_it{it}_"
                for layer in range(t.num_layers):
                    nodes, rows, order = step["inject"][layer]
                    k = write_entries(t.full_to_history_layered[layer], t.history_to_full_layered[layer],
                                      t.checkin_iter[layer], t.history_buffer_layered[layer],
                                      torch.from_numpy(nodes), torch.from_numpy(rows), torch.from_numpy(order), it)
                    out[pre + f"written{layer}"] = np.int64(k)
                batch = types.SimpleNamespace(ptr=torch.from_numpy(b["ptr"]), idx=torch.from_numpy(b["idx"]),
                                              sub_to_full=torch.from_numpy(b["sub_to_full"]),
                                              num_node_in_layer=torch.from_numpy(b["num_node_in_layer"]),
                                              y=torch.zeros(60, dtype=torch.int64), x=None)
                t.lookup(batch.sub_to_full, batch.num_node_in_layer)
                t.history_out = []
                for layer in range(t.num_layers):
                    out[pre + f"sub_to_history{layer}"] = t.sub_to_history[layer].numpy().copy()
                    out[pre + f"compact{layer}"] = t.sub_to_history_layered[layer].numpy().copy()
                    out[pre + f"rows{layer}"] = t.tmp_history_buffer_layered[layer].detach().numpy().copy()
                    assert t.tmp_history_buffer_layered[layer].requires_grad == (case["method"] == "grad")
                    g = torch.from_numpy(step["grads"][layer])
                    h = torch.zeros_like(g).requires_grad_(True)
                    h.grad = g
                    t.history_out.append(h)
                t.evict_history(batch, it)
                hits = []
                for layer in range(t.num_layers):
                    out[pre + f"full_to_history{layer}"] = t.full_to_history_layered[layer].numpy().copy()
                    out[pre + f"history_to_full{layer}"] = t.history_to_full_layered[layer].numpy().copy()
                    out[pre + f"checkin{layer}"] = t.checkin_iter[layer].numpy().copy()
                    hits.append((int((out[pre + f"sub_to_history{layer}"] != -1).sum()),
                                 int((t.history_to_full_layered[layer] != -1).sum())))
                summary.append(hits)
            print(name, "(hits, live entries after eviction) per layer and iteration:", summary)
    path = os.path.join(HERE, "history_table_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
