"""Generates tests/golden/history_cache_golden.npz by running the reference's own
``HistoryCache.update_history`` and ``HistoryCache.lookup_and_load``
(/root/reference/hiscache/history_cache.py:180-356) on CPU tensors.

Run in the build container only (the reference tree is not available elsewhere):

    python tests/golden/gen_history_cache_golden.py          (every fixture; `... fill` the constructor's only)

The reference module's SOURCE TEXT is read from /root/reference, compiled and executed here (no
importlib loader: a loader would prefer a ``__pycache__/*.pyc`` lying beside the source, and would
write one if there was none); its package ``__init__`` (which imports CUDA-only extensions) is not
executed.  Two collaborators that do not
exist here are supplied as small stand-ins, and the fixture records which outputs depend on them:
  * ``hiscache.count_history_reconstruct`` -> this repo's CPU oracle (so ``used_masks`` and everything
    derived from it in lookup_and_load is NOT independent evidence; the id translation, the
    cached-embedding gather with -1 slots and the feature-cache merge are);
  * ``uvm.masked_get(ids, mask)`` -> rows of the feature matrix where the mask is set, zeros elsewhere
    (semantics inferred from history_cache.py:345-349).
``update_history`` needs neither: its golden vectors are produced by the reference code alone.
Only inputs and outputs are stored; no reference source text is copied.
"""
import logging
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, os.path.join(ROOT, "history-cache_amd"))  # synthetic batch generator only
REF = "/root/reference/hiscache/history_cache.py"


def load_reference_class():
    from oracle import hc_oracle as orc

    def count_history_reconstruct(ptr, idx, hmap, num_node, num_seed, num_layer):
        out = orc.count_history_reconstruct(ptr.numpy(), idx.numpy(), hmap.numpy(), num_node, num_seed, num_layer)
        return [torch.from_numpy(m) for m in out]

    pkg = types.ModuleType("hiscache")
    pkg.__path__ = []
    pkg.count_history_reconstruct = count_history_reconstruct
    util = types.ModuleType("hiscache.util")
    util.log = logging.getLogger("reference")
    saved = {k: sys.modules.get(k) for k in ("hiscache", "hiscache.util", "hiscache.history_cache")}
    sys.modules["hiscache"] = pkg
    sys.modules["hiscache.util"] = util
    sys.dont_write_bytecode = True
    mod = types.ModuleType("hiscache.history_cache")
    mod.__file__ = REF
    sys.modules["hiscache.history_cache"] = mod
    with open(REF, "r", encoding="utf-8") as f:
        code = compile(f.read(), REF, "exec")      # the source text itself, never cached bytecode
    exec(code, mod.__dict__)
    for k, v in saved.items():
        if v is None:
            sys.modules.pop(k, None)
        else:
            sys.modules[k] = v
    return mod.HistoryCache


class Store:
    def __init__(self, feats):
        self.buffer = feats

    def masked_get(self, ids, mask):
        out = torch.zeros((ids.shape[0], self.buffer.shape[1]), dtype=torch.float32)
        out[mask] = self.buffer[ids[mask]]
        return out


def main():
    from helpers import layered_batch
    HistoryCache = load_reference_class()
    rng = np.random.default_rng(2024)
    N, Fin, H, n_iter = 1500, 8, 12, 7
    buffer_floats = 24 * 400                      # 1200 feature slots, 800 embedding slots
    feats = torch.from_numpy(rng.standard_normal((N, Fin)).astype(np.float32))
    hot = torch.from_numpy(rng.permutation(N).astype(np.int64))

    c = HistoryCache.__new__(HistoryCache)         # __init__ needs a GPU and dataset files
    c.in_channels, c.hidden_channels, c.total_num_node = Fin, H, N
    c.device = torch.device("cpu")
    c.method, c.rate, c.staleness_thres, c.start_history = "grad", 0.6, 4, 0
    c.feat_mode, c.distributed_store = "history_uvm", False
    c.uvm = Store(feats)
    c.header, c.glb_iter, c.num_stored_history = 0, 0, 0
    c.produced_embedding, c.used_masks = None, None
    # the state HistoryCache.allocate/fill build (history_cache.py:42-46, 110-116, 134-139, 156-167)
    c.full2embed = torch.ones([2 * N + 1], dtype=torch.int64) * -1
    c.buffer = torch.zeros(buffer_floats)
    c.embed2full = torch.ones(buffer_floats // H, dtype=torch.int64) * -1
    n_feat = buffer_floats // Fin
    cache_ids = hot[-n_feat:]
    c.feat2full = cache_ids + N
    c.full2embed[c.feat2full] = torch.arange(0, n_feat)
    c.buffer.view(-1, Fin)[-n_feat:] = feats[cache_ids]

    out = {"N": N, "Fin": Fin, "H": H, "buffer_floats": buffer_floats, "features": feats.numpy(), "hot": hot.numpy(),
           "rate": 0.6, "staleness_thres": 4, "n_iter": n_iter}
    high = 0
    for it in range(1, n_iter + 1):
        b = layered_batch(rng, N, 20, [5, 4])
        batch = types.SimpleNamespace(ptr=torch.from_numpy(b["ptr"]), idx=torch.from_numpy(b["idx"]),
                                      sub_to_full=torch.from_numpy(b["sub_to_full"]),
                                      num_node_in_layer=torch.from_numpy(b["num_node_in_layer"]),
                                      y=torch.zeros(20, dtype=torch.int64), x=None)
        c.lookup_and_load(batch, 2)
        n1 = int(b["num_node_in_layer"][1])
        emb = rng.standard_normal((n1, H)).astype(np.float32)
        grad = (rng.standard_normal((n1, H)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)
        pe = torch.from_numpy(emb.copy()).requires_grad_(True)
        pe.grad = torch.from_numpy(grad.copy())
        c.produced_embedding = pe
        pre = f"it{it}_"
        for k in ("ptr", "idx", "sub_to_full", "num_node_in_layer"):
            out[pre + k] = b[k]
        out[pre + "emb"], out[pre + "grad"] = emb, grad
        out[pre + "sub2embed"] = c.sub2embed.numpy().copy()
        out[pre + "sub2feat"] = c.sub2feat.numpy().copy()
        out[pre + "cached_embedding"] = c.cached_embedding.numpy().copy()
        out[pre + "x"] = batch.x.numpy().copy()
        c.update_history(batch, it)
        out[pre + "full2embed"] = c.full2embed.numpy().copy()
        out[pre + "embed2full"] = c.embed2full.numpy().copy()
        out[pre + "header"] = np.int64(c.header)
        high = max(high, c.header)
        out[pre + "buffer_front"] = c.buffer.numpy()[: high * H].copy()   # every embedding row written so far
    np.savez_compressed(os.path.join(HERE, "history_cache_golden.npz"), **out)
    print("wrote", os.path.join(HERE, "history_cache_golden.npz"), "headers:",
          [int(out[f"it{i}_header"]) for i in range(1, n_iter + 1)])


# ---- the admission at the widths of the plumbing configuration -------------------------------------------
# 100 000 nodes, 128-wide features and embeddings, about 10 000 one-hop rows per batch, rate 0.5, five
# iterations with a staleness refresh.  The inputs are rebuilt from seeds by tests/helpers.py (exact_rows,
# affine_ids); the fixture keeps the seeds and what the reference's update_history made of them: the record
# mask, the reference's own scores and threshold (so that a test can count the rows at the knife edge should a
# mask ever differ), the header, and digests of the maps and of the stored rows.
WIDE_CASES = {
    "": dict(N=100_000, Fin=128, H=128, n1=10_000, n_seed=1000, rate=0.5, staleness_thres=3, n_iter=5,
             buffer_floats=128 * 24_000, seed=77),
    # the hidden width of the papers100M- and mag240M-shaped configurations
    "_h256": dict(N=100_000, Fin=128, H=256, n1=10_000, n_seed=1000, rate=0.5, staleness_thres=3, n_iter=5,
                  buffer_floats=256 * 20_000, seed=78),
}


def wide_inputs(w, it):
    """(sub_to_full[:n1], embedding rows, gradient rows) of iteration `it` (1-based)."""
    from helpers import affine_ids, exact_rows
    ids = affine_ids(w["N"], w["n1"], 7919 + 20 * it, 31 * it)       # overlaps the earlier batches in part
    emb = exact_rows(w["seed"] + 100 * it, w["n1"], w["H"], octaves=1)
    grad = exact_rows(w["seed"] + 100 * it + 1, w["n1"], w["H"])
    return ids, emb, grad


def digest(a):
    import hashlib
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), dtype=np.uint8).copy()


def main_wide(suffix):
    from helpers import exact_rows
    HistoryCache = load_reference_class()
    w = WIDE_CASES[suffix]
    N, Fin, H = w["N"], w["Fin"], w["H"]
    feats = torch.from_numpy(exact_rows(w["seed"], N, Fin, octaves=1))
    hot = torch.from_numpy(((np.arange(N, dtype=np.int64) * 48271 + 11) % N).astype(np.int64))

    c = HistoryCache.__new__(HistoryCache)
    c.in_channels, c.hidden_channels, c.total_num_node = Fin, H, N
    c.device = torch.device("cpu")
    c.method, c.rate, c.staleness_thres, c.start_history = "grad", w["rate"], w["staleness_thres"], 0
    c.feat_mode, c.distributed_store = "history_uvm", False
    c.header, c.glb_iter, c.num_stored_history = 0, 0, 0
    c.full2embed = torch.ones([2 * N + 1], dtype=torch.int64) * -1
    c.buffer = torch.zeros(w["buffer_floats"])
    c.embed2full = torch.ones(w["buffer_floats"] // H, dtype=torch.int64) * -1
    n_feat = w["buffer_floats"] // Fin
    cache_ids = hot[-n_feat:]
    c.feat2full = cache_ids + N
    c.full2embed[c.feat2full] = torch.arange(0, n_feat)
    c.buffer.view(-1, Fin)[-n_feat:] = feats[cache_ids]

    out = {k: np.asarray(v) for k, v in w.items()}
    high = 0
    for it in range(1, w["n_iter"] + 1):
        ids, emb, grad = wide_inputs(w, it)
        batch = types.SimpleNamespace(sub_to_full=torch.from_numpy(ids),
                                      num_node_in_layer=torch.tensor([w["n_seed"], w["n1"]]))
        # what lookup_and_load leaves behind for update_history (history_cache.py:307-310), seeds excluded as there
        c.sub2embed = c.full2embed[batch.sub_to_full[: w["n1"]]]
        pe = torch.from_numpy(emb.copy()).requires_grad_(True)
        pe.grad = torch.from_numpy(grad.copy())
        c.produced_embedding = pe
        score = pe.grad.norm(dim=1)                                   # the reference's own expressions
        thres = torch.quantile(score, w["rate"])                       # (history_cache.py:205, 211)
        before = c.full2embed[batch.sub_to_full[: w["n1"]]].clone()
        header_before = 0 if it % w["staleness_thres"] == 0 else c.header
        c.update_history(batch, it)
        after = c.full2embed[batch.sub_to_full[: w["n1"]]]
        recorded = (after >= header_before) & (after < c.header) & (before == -1)
        pre = f"it{it}_"
        out[pre + "record_mask"] = np.packbits(recorded.numpy())
        out[pre + "ref_score"] = score.numpy().copy()
        out[pre + "ref_thres"] = np.float32(thres)
        out[pre + "header"] = np.int64(c.header)
        high = max(high, c.header)
        out[pre + "full2embed_sha256"] = digest(c.full2embed.numpy())
        out[pre + "embed2full_sha256"] = digest(c.embed2full.numpy())
        out[pre + "buffer_front_sha256"] = digest(c.buffer.numpy()[: high * H])
        out[pre + "rows_stored"] = np.int64(high)
    path = os.path.join(HERE, "history_cache_golden_wide%s.npz" % suffix)
    np.savez_compressed(path, **out)
    print("wrote", path, "headers:", [int(out[f"it{i}_header"]) for i in range(1, w["n_iter"] + 1)],
          "bytes:", os.path.getsize(path))


# ---- the constructor: allocate() and fill() -------------------------------------------------------------
# HistoryCache.__init__ -> allocate() -> fill() (history_cache.py:12-62, 95-178) run as they are, on the CPU,
# from dataset files written here (num_nodes.txt, sorted_indices.dat).  allocate() asks the CUDA runtime for the
# free device memory; there is none here, so that one query answers 64 GiB for the duration of the call (the
# limit in the configuration then decides the size, as in every run of the reference with a limit).  The buffer
# that allocate() makes is uninitialised: only the rows that fill() writes are kept.
FILL_CASES = {
    "part": dict(N=1500, Fin=8, H=12, limit_gb=1e-5, seed=41),       # room for 336 feature rows of 1500
    "all": dict(N=200, Fin=8, H=12, limit_gb=1e-5, seed=42),         # room for more rows than there are nodes
    "wide": dict(N=3000, Fin=16, H=24, limit_gb=1e-4, seed=43),
}


def fill_inputs(c):
    """(features, node ids sorted coldest to hottest) of a fill case, rebuilt from its seed."""
    from helpers import exact_rows
    feats = exact_rows(c["seed"], c["N"], c["Fin"], octaves=2)
    hot = np.random.default_rng(c["seed"]).permutation(c["N"]).astype(np.int64)
    return feats, hot


def eval_ids(c):
    """Node ids of a fill case's evaluation lookup, rebuilt from its seed (repeated ids included)."""
    return np.random.default_rng(c["seed"] + 100).integers(0, c["N"], size=min(c["N"], 700)).astype(np.int64)


def main_fill():
    import tempfile
    sys.path.insert(0, os.path.join(ROOT, "history-cache_amd"))
    from hiscache.util import make_config
    HistoryCache = load_reference_class()
    out = {}
    probe = torch.cuda.mem_get_info
    torch.cuda.mem_get_info = lambda *a, **k: (64 << 30, 64 << 30)
    try:
        for name, c in FILL_CASES.items():
            feats, hot = fill_inputs(c)
            with tempfile.TemporaryDirectory() as root:
                os.makedirs(os.path.join(root, "processed"))
                with open(os.path.join(root, "processed", "num_nodes.txt"), "w") as f:
                    f.write("%d\n" % c["N"])
                hot.tofile(os.path.join(root, "processed", "sorted_indices.dat"))
                cfg = make_config(c["Fin"], 5, c["H"], 2, method="grad", rate=0.5, staleness_thres=4,
                                  limit=c["limit_gb"], device="cpu", path=root)
                cache = HistoryCache(Store(torch.from_numpy(feats)), cfg, "history_uvm")
            n_cached = min(cache.overall_feat_num, c["N"])
            pre = name + "_"
            out[pre + "hot"] = hot
            out[pre + "max_buffer_byte"] = np.int64(cache.max_buffer_byte)
            out[pre + "overall_feat_num"] = np.int64(cache.overall_feat_num)
            out[pre + "overall_embed_num"] = np.int64(cache.overall_embed_num)
            out[pre + "buffer_floats"] = np.int64(cache.buffer.shape[0])
            out[pre + "feat2full"] = cache.feat2full.numpy().copy()
            out[pre + "full2embed"] = cache.full2embed.numpy().copy()
            out[pre + "embed2full"] = cache.embed2full.numpy().copy()
            out[pre + "feature_rows"] = cache.buffer.view(-1, c["Fin"])[-n_cached:].numpy().copy()
            out[pre + "header"] = np.int64(cache.header)
            # the evaluation lookup (history_cache.py:276-288) on the cache as fill() left it: nodes with and
            # without a cached feature row, the store stand-in serving the others
            ids = eval_ids(c)
            batch = types.SimpleNamespace(sub_to_full=torch.from_numpy(ids), x=None)
            cache.lookup_and_load(batch, 2, feature_cache_only=True)
            out[pre + "eval_sub2feat"] = cache.sub2feat.numpy().copy()
            out[pre + "eval_x"] = batch.x.numpy().copy()
            print(name, "buffer floats", cache.buffer.shape[0], "feature slots", cache.overall_feat_num,
                  "cached", n_cached, "evaluation lookup: rows from the cache",
                  int((cache.sub2feat != -1).sum()), "of", len(ids))
    finally:
        torch.cuda.mem_get_info = probe
    path = os.path.join(HERE, "history_cache_fill_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    if sys.argv[1:] == ["fill"]:
        main_fill()
    else:
        main()
        for suffix in WIDE_CASES:
            main_wide(suffix)
        main_fill()
