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


# ---- the admission at the plumbing configuration's widths (128-wide rows, 10 000 one-hop rows per batch) ----
EXACT_ROWS_DIGEST = "7df0f62c50da8be0041fa1c1f53b8388f7e865cc1a8e791003906c644f65e219"
WIDE = {h: os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "history_cache_golden_wide%s.npz" % sfx)
        for h, sfx in ((128, ""), (256, "_h256"))}


def wide_inputs(g, it):
    from helpers import affine_ids, exact_rows
    N, n1, H, seed = int(g["N"]), int(g["n1"]), int(g["H"]), int(g["seed"])
    ids = affine_ids(N, n1, 7919 + 20 * it, 31 * it)
    emb = exact_rows(seed + 100 * it, n1, H, octaves=1)
    grad = exact_rows(seed + 100 * it + 1, n1, H)
    return ids, emb, grad


def sha256_of(t):
    import hashlib
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(t).tobytes()).digest(), dtype=np.uint8)


def knife_edge_rows(score, thres):
    """Rows whose score lies within 2 ulp of the threshold: the only rows whose side of `score < thres` can
    depend on the order in which a row's squares were added."""
    ulp = np.spacing(np.float32(abs(thres)))
    return int((np.abs(score.astype(np.float64) - float(thres)) <= 2.0 * float(ulp)).sum())


def check_wide_iteration(g, it, mask, score, header, full2embed, embed2full, buffer):
    pre = f"it{it}_"
    n1, H = int(g["n1"]), int(g["H"])
    want_mask = np.unpackbits(g[pre + "record_mask"])[:n1].astype(bool)
    differ = int((mask != want_mask).sum())
    # should a mask ever differ, say how many rows sit at the knife edge of either side's threshold
    edge = knife_edge_rows(g[pre + "ref_score"], g[pre + "ref_thres"]) + knife_edge_rows(score, g[pre + "ref_thres"])
    assert differ == 0, f"iteration {it}: {differ} rows of the record mask differ; {edge} rows within 2 ulp of the threshold"
    assert header == int(g[pre + "header"])
    np.testing.assert_array_equal(sha256_of(full2embed), g[pre + "full2embed_sha256"])
    np.testing.assert_array_equal(sha256_of(embed2full), g[pre + "embed2full_sha256"])
    rows = int(g[pre + "rows_stored"])
    np.testing.assert_array_equal(sha256_of(buffer[: rows * H]), g[pre + "buffer_front_sha256"])


def test_exact_rows_are_rebuilt_bit_for_bit():
    """The fixture's inputs come from integer hashes: a known digest pins them on any machine."""
    from helpers import affine_ids, exact_rows
    r = exact_rows(77, 300, 128)
    assert r.dtype == np.float32 and np.isfinite(r).all() and (np.abs(r) < 4).all()
    norms = np.linalg.norm(r.astype(np.float64), axis=1)
    assert norms.max() / norms.min() > 500                   # rows spread over several octaves
    assert sha256_of(r).tobytes().hex() == EXACT_ROWS_DIGEST
    ids = affine_ids(100_000, 10_000, 7939, 31)
    assert len(np.unique(ids)) == 10_000


@pytest.mark.parametrize("hidden", [128, 256])
def test_oracle_reproduces_reference_vectors_at_real_width(orc, hidden):
    """oracle.host_model.update_history with the oracle's row scores (the kernel's lane order) against what the
    reference's grad.norm(dim=1) + torch.quantile + masking recorded: masks, maps, header, stored rows."""
    from helpers import exact_rows
    from oracle import host_model
    g = np.load(WIDE[hidden], allow_pickle=False)
    N, Fin, H, n1 = int(g["N"]), int(g["Fin"]), int(g["H"]), int(g["n1"])
    feats = torch.from_numpy(exact_rows(int(g["seed"]), N, Fin, octaves=1))
    hot = ((np.arange(N, dtype=np.int64) * 48271 + 11) % N).astype(np.int64)
    st = host_model.new_cache_state(N, Fin, H, int(g["buffer_floats"]), hot, feats)
    for it in range(1, int(g["n_iter"]) + 1):
        ids, emb, grad = wide_inputs(g, it)
        sub_to_full = torch.from_numpy(ids)
        sub2embed = st.full2embed[sub_to_full[:n1]]
        score = orc.row_scores(grad)
        mask, _ = host_model.update_history(st, sub_to_full, sub2embed, torch.from_numpy(emb), torch.from_numpy(score),
                                            float(g["rate"]), int(g["staleness_thres"]), it)
        check_wide_iteration(g, it, mask.numpy(), score, st.header, st.full2embed.numpy(), st.embed2full.numpy(),
                             st.buffer.numpy())


@pytest.mark.gpu
@pytest.mark.parametrize("hidden", [128, 256])
def test_gpu_cache_reproduces_reference_vectors_at_real_width(hidden):
    """The GPU HistoryCache.update_history (hc_row_scores + hc_quantile_threshold + hc_cache_append) at 128- and
    256-wide rows and 10 000 rows per batch against the reference's own admission, exactly."""
    from helpers import exact_rows
    from hiscache import HistoryCache, PinnedFeatureStore, make_config
    dev = "cuda:0"
    g = np.load(WIDE[hidden], allow_pickle=False)
    N, Fin, H, n1 = int(g["N"]), int(g["Fin"]), int(g["H"]), int(g["n1"])
    feats = torch.from_numpy(exact_rows(int(g["seed"]), N, Fin, octaves=1))
    hot = ((np.arange(N, dtype=np.int64) * 48271 + 11) % N).astype(np.int64)
    cfg = make_config(Fin, 5, H, 2, method="grad", rate=float(g["rate"]), staleness_thres=int(g["staleness_thres"]),
                      device=dev)
    cache = HistoryCache(PinnedFeatureStore(feats, device=dev), cfg, "history_uvm", total_num_node=N,
                         buffer_bytes=int(g["buffer_floats"]) * 4, hot_ids=hot)
    for it in range(1, int(g["n_iter"]) + 1):
        ids, emb, grad = wide_inputs(g, it)
        batch = SimpleNamespace(sub_to_full=torch.from_numpy(ids).to(dev),
                                num_node_in_layer=torch.tensor([int(g["n_seed"]), n1]))
        # what lookup_and_load leaves for update_history (reference history_cache.py:307-310)
        cache.sub2embed = cache.full2embed[batch.sub_to_full[:n1]]
        pe = torch.from_numpy(emb).to(dev).requires_grad_(True)
        pe.grad = torch.from_numpy(grad).to(dev)
        cache.produced_embedding = pe
        cache.update_history(batch, it)
        check_wide_iteration(g, it, cache.last_record_mask.cpu().numpy().astype(bool), cache.last_score.cpu().numpy(),
                             cache.header, cache.full2embed.cpu().numpy(), cache.embed2full.cpu().numpy(),
                             cache.buffer.cpu().numpy())


# ---- the constructor: allocate() and fill() as the reference ran them ---------------------------------------
FILL = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "history_cache_fill_golden.npz")
FILL_CASES = {                      # tests/golden/gen_history_cache_golden.py:FILL_CASES
    "part": dict(N=1500, Fin=8, H=12, limit_gb=1e-5, seed=41),
    "all": dict(N=200, Fin=8, H=12, limit_gb=1e-5, seed=42),
    "wide": dict(N=3000, Fin=16, H=24, limit_gb=1e-4, seed=43),
}


def fill_inputs(c, g, name):
    from helpers import exact_rows
    feats = exact_rows(c["seed"], c["N"], c["Fin"], octaves=2)
    hot = np.random.default_rng(c["seed"]).permutation(c["N"]).astype(np.int64)
    np.testing.assert_array_equal(hot, g[name + "_hot"], err_msg="the case's inputs are not the fixture's")
    return feats, hot


def eval_ids(c):
    """tests/golden/gen_history_cache_golden.py:eval_ids"""
    return np.random.default_rng(c["seed"] + 100).integers(0, c["N"], size=min(c["N"], 700)).astype(np.int64)


def check_fill(name, g, N, Fin, buffer_floats, feat2full, full2embed, embed2full, buffer, header):
    """The reference keeps only the cached block in feat2full; here it is slot-indexed with -1 in the empty
    slots in front, so its tail is compared."""
    pre = name + "_"
    n_cached = len(g[pre + "feat2full"])
    assert buffer_floats == int(g[pre + "buffer_floats"])
    np.testing.assert_array_equal(feat2full[-n_cached:], g[pre + "feat2full"])
    assert (feat2full[:-n_cached] == -1).all()
    np.testing.assert_array_equal(full2embed, g[pre + "full2embed"])
    np.testing.assert_array_equal(embed2full, g[pre + "embed2full"])
    slots = buffer_floats // Fin
    np.testing.assert_array_equal(buffer[: slots * Fin].reshape(slots, Fin)[-n_cached:], g[pre + "feature_rows"])
    assert header == int(g[pre + "header"]) == 0


@pytest.mark.parametrize("name", list(FILL_CASES))
def test_oracle_reproduces_reference_constructor(name):
    from oracle import host_model
    g = np.load(FILL, allow_pickle=False)
    c = FILL_CASES[name]
    feats, hot = fill_inputs(c, g, name)
    floats = int(g[name + "_buffer_floats"])
    st = host_model.new_cache_state(c["N"], c["Fin"], c["H"], floats, hot, torch.from_numpy(feats))
    assert floats // c["Fin"] == int(g[name + "_overall_feat_num"])
    assert floats // c["H"] == int(g[name + "_overall_embed_num"])
    check_fill(name, g, c["N"], c["Fin"], floats, st.feat2full.numpy(), st.full2embed.numpy(), st.embed2full.numpy(),
               st.buffer.numpy(), st.header)
    # the reference's evaluation lookup (feature_cache_only=True) on the cache as its fill() left it
    sub2feat, x = host_model.lookup_feature_cache_only(st, torch.from_numpy(eval_ids(c)), torch.from_numpy(feats))
    np.testing.assert_array_equal(sub2feat.numpy(), g[name + "_eval_sub2feat"])
    np.testing.assert_array_equal(x.numpy(), g[name + "_eval_x"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(FILL_CASES))
def test_gpu_cache_reproduces_reference_constructor(name, tmp_path):
    """HistoryCache.__init__ from dataset files (num_nodes.txt, sorted_indices.dat), sized by the
    configuration's limit as the reference sizes it."""
    from hiscache import HistoryCache, PinnedFeatureStore, make_config
    dev = "cuda:0"
    g = np.load(FILL, allow_pickle=False)
    c = FILL_CASES[name]
    feats, hot = fill_inputs(c, g, name)
    os.makedirs(tmp_path / "processed")
    (tmp_path / "processed" / "num_nodes.txt").write_text("%d\n" % c["N"])
    hot.tofile(str(tmp_path / "processed" / "sorted_indices.dat"))
    cfg = make_config(c["Fin"], 5, c["H"], 2, method="grad", rate=0.5, staleness_thres=4, limit=c["limit_gb"],
                      device=dev, path=str(tmp_path))
    cache = HistoryCache(PinnedFeatureStore(torch.from_numpy(feats), device=dev), cfg, "history_uvm")
    assert cache.total_num_node == c["N"]
    assert cache.max_buffer_byte == int(g[name + "_max_buffer_byte"])
    assert cache.overall_feat_num == int(g[name + "_overall_feat_num"])
    assert cache.overall_embed_num == int(g[name + "_overall_embed_num"])
    check_fill(name, g, c["N"], c["Fin"], cache.buffer.numel(), cache.feat2full.cpu().numpy(),
               cache.full2embed.cpu().numpy(), cache.embed2full.cpu().numpy(), cache.buffer.cpu().numpy(), cache.header)
    # the evaluation lookup: the reference's own batch.x and feature slots for the same ids
    from types import SimpleNamespace
    batch = SimpleNamespace(sub_to_full=torch.from_numpy(eval_ids(c)).to(dev), x=None)
    cache.lookup_and_load(batch, 2, feature_cache_only=True)
    np.testing.assert_array_equal(cache.sub2feat.cpu().numpy(), g[name + "_eval_sub2feat"])
    np.testing.assert_array_equal(batch.x.cpu().numpy(), g[name + "_eval_x"])
    assert int((cache.sub2feat != -1).sum()) > 0 and cache.used_masks is None
