"""Golden vectors produced by the reference's own HistoryCache.update_history / lookup_and_load
(tests/golden/gen_history_cache_golden.py ran /root/reference/hiscache/history_cache.py on CPU tensors).
The CPU restatement (oracle.host_model) and the GPU implementation must both reproduce them:
masks, maps, header and stored rows exactly."""
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "history_cache_golden.npz")


def load():
    return np.load(GOLD, allow_pickle=False)


def batch_of(g, it, device):
    pre = f"it{it}_"
    t = lambda k: torch.from_numpy(g[pre + k]).to(device)
    return SimpleNamespace(ptr=t("ptr"), idx=t("idx"), sub_to_full=t("sub_to_full"),
                           num_node_in_layer=torch.from_numpy(g[pre + "num_node_in_layer"]),
                           y=torch.zeros(int(g[pre + "num_node_in_layer"][0]), dtype=torch.int64, device=device), x=None)


def test_oracle_reproduces_reference_vectors(orc):
    from oracle import host_model
    g = load()
    N, Fin, H = int(g["N"]), int(g["Fin"]), int(g["H"])
    feats = torch.from_numpy(g["features"])
    st = host_model.new_cache_state(N, Fin, H, int(g["buffer_floats"]), g["hot"], feats)
    for it in range(1, int(g["n_iter"]) + 1):
        pre = f"it{it}_"
        batch = batch_of(g, it, "cpu")
        out = host_model.lookup_and_load(st, batch, 2, feats)
        np.testing.assert_array_equal(out.sub2embed.numpy(), g[pre + "sub2embed"])
        np.testing.assert_array_equal(out.sub2feat.numpy(), g[pre + "sub2feat"])
        np.testing.assert_array_equal(out.cached_embedding.numpy(), g[pre + "cached_embedding"])
        np.testing.assert_array_equal(out.x.numpy(), g[pre + "x"])
        score = torch.from_numpy(orc.row_scores(g[pre + "grad"]))
        host_model.update_history(st, batch.sub_to_full, out.sub2embed, torch.from_numpy(g[pre + "emb"]), score,
                                  float(g["rate"]), int(g["staleness_thres"]), it)
        np.testing.assert_array_equal(st.full2embed.numpy(), g[pre + "full2embed"])
        np.testing.assert_array_equal(st.embed2full.numpy(), g[pre + "embed2full"])
        assert st.header == int(g[pre + "header"])
        front = g[pre + "buffer_front"]
        np.testing.assert_array_equal(st.buffer.numpy()[: front.size], front)


@pytest.mark.gpu
def test_gpu_cache_reproduces_reference_vectors():
    from hiscache import HistoryCache, PinnedFeatureStore, make_config
    dev = "cuda:0"
    g = load()
    N, Fin, H = int(g["N"]), int(g["Fin"]), int(g["H"])
    feats = torch.from_numpy(g["features"])
    cfg = make_config(Fin, 5, H, 2, method="grad", rate=float(g["rate"]), staleness_thres=int(g["staleness_thres"]),
                      device=dev)
    cache = HistoryCache(PinnedFeatureStore(feats, device=dev), cfg, "history_uvm", total_num_node=N,
                         buffer_bytes=int(g["buffer_floats"]) * 4, hot_ids=g["hot"])
    for it in range(1, int(g["n_iter"]) + 1):
        pre = f"it{it}_"
        batch = batch_of(g, it, dev)
        cache.lookup_and_load(batch, 2)
        np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), g[pre + "sub2embed"])
        np.testing.assert_array_equal(cache.sub2feat.cpu().numpy(), g[pre + "sub2feat"])
        np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), g[pre + "cached_embedding"])
        np.testing.assert_array_equal(batch.x.cpu().numpy(), g[pre + "x"])
        pe = torch.from_numpy(g[pre + "emb"]).to(dev).requires_grad_(True)
        pe.grad = torch.from_numpy(g[pre + "grad"]).to(dev)
        cache.produced_embedding = pe
        cache.update_history(batch, it)
        np.testing.assert_array_equal(cache.full2embed.cpu().numpy(), g[pre + "full2embed"])
        np.testing.assert_array_equal(cache.embed2full.cpu().numpy(), g[pre + "embed2full"])
        assert cache.header == int(g[pre + "header"])
        front = g[pre + "buffer_front"]
        np.testing.assert_array_equal(cache.buffer.cpu().numpy()[: front.size], front)
