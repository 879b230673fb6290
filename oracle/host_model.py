"""Torch-CPU restatement of the reference's host-side cache policy.

TEST INFRASTRUCTURE ONLY (see hc_oracle.c).  Statement by statement it follows
``HistoryCache.update_history`` / ``lookup_and_load``
(/root/reference/hiscache/history_cache.py:180-255, 275-356) and the lookup and eviction rules of
``HistoryTable`` (/root/reference/hiscache/history_table.py:94-125, 189-251), on CPU tensors, with the
kernel calls replaced by the C oracle.  State lives in a plain object so tests can compare every
tensor with the GPU implementation.  Pinned by vectors that the reference's own code produced
(tests/golden: the cache's two entry points, its constructor and its evaluation lookup, the table's lookup and
evictions).
"""
import math
from types import SimpleNamespace

import numpy as np
import torch

from . import hc_oracle as orc


def quantile_threshold(score, rate):
    """The admission threshold with the build's documented arithmetic (separately rounded fp32
    operations; mathematically torch.quantile(score, rate), history_cache.py:211)."""
    s = np.sort(np.asarray(score, np.float32).reshape(-1))
    n = s.size
    if np.isnan(s).any():            # torch.quantile answers NaN when any score is NaN (history_cache.py:211)
        return np.float32("nan")
    pos = np.float32(np.float32(rate) * np.float32(n - 1))   # torch.quantile ranks in the data's dtype
    lo = min(int(np.floor(pos)), n - 1)
    hi = min(lo + 1, n - 1)
    w = np.float32(pos - np.float32(lo))
    a, b = s[lo], s[hi]
    d = np.float32(b - a)
    if w < np.float32(0.5):
        return np.float32(a + np.float32(d * w))
    return np.float32(b - np.float32(d * np.float32(np.float32(1.0) - w)))


def new_cache_state(total_num_node, in_channels, hidden, buffer_floats, hot_ids, features):
    """Mirror of HistoryCache.__init__/allocate/fill (history_cache.py:42-63, 95-178) with sizes
    given explicitly.  ``feat2full`` is slot-indexed (-1 = empty slot)."""
    N = total_num_node
    st = SimpleNamespace()
    st.N, st.Fin, st.H = N, in_channels, hidden
    st.full2embed = torch.full((2 * N + 1,), -1, dtype=torch.int64)
    st.buffer = torch.zeros(buffer_floats, dtype=torch.float32)
    st.embed2full = torch.full((buffer_floats // hidden,), -1, dtype=torch.int64)
    n_feat_slots = buffer_floats // in_channels
    hot = torch.as_tensor(hot_ids, dtype=torch.int64)
    cache_ids = hot if n_feat_slots > N else (hot[-n_feat_slots:] if n_feat_slots > 0 else hot[:0])
    first = n_feat_slots - cache_ids.numel()
    st.feat2full = torch.full((n_feat_slots,), -1, dtype=torch.int64)
    st.feat2full[first:] = cache_ids + N
    st.full2embed[cache_ids + N] = torch.arange(first, n_feat_slots)
    if cache_ids.numel():
        st.buffer.view(-1, in_channels)[first:n_feat_slots] = features[cache_ids].to(torch.float32)
    st.header = 0
    st.glb_iter = 0
    return st


def lookup_and_load(st, batch, num_layer, features):
    """history_cache.py:306-351.  ``features`` is the full host feature matrix (the role of
    uvm.masked_get: rows where the mask is false are zero).  Returns a namespace with
    sub2embed, cached_embedding, sub2feat, used_masks, load_mask, x."""
    n1 = int(batch.num_node_in_layer[1])
    sub_to_full = batch.sub_to_full
    layer1_nodes = sub_to_full[:n1]
    sub2embed = st.full2embed[layer1_nodes]
    cached_embedding = st.buffer.view(-1, st.H)[sub2embed]
    sub2feat = st.full2embed[sub_to_full + st.N]
    used = orc.count_history_reconstruct(batch.ptr.numpy(), batch.idx.numpy(), sub2embed.numpy(),
                                         sub_to_full.shape[0], batch.y.shape[0], num_layer)
    used_masks = [torch.from_numpy(m) for m in used]
    hit_feat_mask = sub2feat != -1
    load_mask = torch.logical_and(used_masks[0], ~hit_feat_mask)
    st.glb_iter += 1
    x = torch.zeros((sub_to_full.shape[0], st.Fin), dtype=torch.float32)
    x[load_mask] = features[sub_to_full[load_mask]].to(torch.float32)
    cached_feat = st.buffer.view(-1, st.Fin)[sub2feat]
    cached_feat[~hit_feat_mask] = 0
    x += cached_feat
    return SimpleNamespace(sub2embed=sub2embed, cached_embedding=cached_embedding, sub2feat=sub2feat,
                           used_masks=used_masks, load_mask=load_mask, x=x)


def lookup_feature_cache_only(st, sub_to_full, features):
    """history_cache.py:276-288, the evaluation lookup: feature-cache hits from the buffer's tail, every other
    row from the host matrix.  Pinned by the reference's own run (history_cache_fill_golden.npz).
    Returns (sub2feat, x)."""
    sub2feat = st.full2embed[sub_to_full + st.N]
    load_mask = sub2feat == -1
    x = torch.zeros((sub_to_full.shape[0], st.Fin), dtype=torch.float32)
    x[load_mask] = features[sub_to_full[load_mask]].to(torch.float32)
    cached_feat = st.buffer.view(-1, st.Fin)[sub2feat]
    cached_feat[load_mask] = 0
    x += cached_feat
    return sub2feat, x


def update_history(st, sub_to_full, sub2embed, produced_embedding, score, rate, staleness_thres,
                   glb_iter):
    """history_cache.py:188-254 with the score given (the caller computes the row norms with the
    oracle's summation order).  Rows that would land beyond the buffer are dropped (the reference
    raises there).  Returns (record_mask, thres)."""
    num_node = produced_embedding.shape[0]
    if (glb_iter % staleness_thres) == 0:
        st.header = 0
    thres = quantile_threshold(score.numpy(), rate)
    record_mask = torch.logical_and(score < float(thres), sub2embed == -1)
    embed_to_record = produced_embedding[record_mask]
    capacity = st.embed2full.numel()
    room = max(0, capacity - st.header)
    keep = min(embed_to_record.shape[0], room)
    change_id_all = sub_to_full[:num_node][record_mask]
    embed_to_record = embed_to_record[:keep]
    change_id = change_id_all[:keep]
    num_to_record = keep
    st.buffer.view(-1, st.H)[st.header:st.header + num_to_record] = embed_to_record
    # invalidate the previously cached features that the new rows overlap
    begin = st.header * st.H // st.Fin
    end = math.ceil((st.header + num_to_record) * st.H / st.Fin)
    f = st.feat2full[begin:end]
    st.full2embed[f[f >= 0]] = -1
    # invalidate the embeddings that are about to be overwritten
    invalid_fulls = st.embed2full[st.header:st.header + num_to_record]
    change_area = st.full2embed[invalid_fulls]
    change_area[torch.logical_and(change_area >= st.header,
                                  change_area < st.header + num_to_record)] = -1
    st.full2embed[invalid_fulls] = change_area
    new_id = torch.arange(st.header, st.header + num_to_record)
    st.full2embed[change_id] = new_id
    st.embed2full[st.header:st.header + num_to_record] = change_id
    st.header += num_to_record
    return record_mask, thres


def table_lookup(full_to_history, history_buffer, sub_to_full, num_node, num_seed):
    """history_table.py:100-125 for one layer: the slot of each of the first ``num_node`` sub-graph nodes
    (-1 for the seeds and for nodes without an entry), the rows of the hits in node order, and the compact
    ids [-1, 0, -1, 1, ...] that point into those rows."""
    sub_to_history = full_to_history[sub_to_full[:num_node]].clone()
    sub_to_history[:num_seed] = -1
    mask = sub_to_history != -1
    rows = history_buffer[sub_to_history[mask]]
    compact = torch.full((num_node,), -1, dtype=torch.int64)
    compact[mask] = torch.arange(int(mask.sum()))
    return sub_to_history, rows, compact


def evict_by_staleness(checkin, history_to_full, full_to_history, glb_iter, staleness_thres):
    """history_table.py:193-200 for one layer, in place."""
    stale_iter = glb_iter - staleness_thres
    hist_id = torch.logical_and(-1 < checkin, checkin <= stale_iter).nonzero().view(-1)
    full_id = history_to_full[hist_id]
    checkin[hist_id] = -1
    history_to_full[hist_id] = -1
    full_to_history[full_id] = -1


def evict_by_both(checkin, history_to_full, full_to_history, sub_to_history, score, rate, glb_iter,
                  staleness_thres):
    """history_table.py:230-251 for one layer, in place: rows of the batch whose score reaches
    quantile(score, 1 - rate) give up their slot, then the staleness rule runs."""
    thres = quantile_threshold(score, 1 - rate)
    to_evict = torch.masked_select(sub_to_history, score >= thres)
    to_evict = to_evict[to_evict != -1]
    full_to_history[history_to_full[to_evict]] = -1
    history_to_full[to_evict] = -1
    checkin[to_evict] = -1
    evict_by_staleness(checkin, history_to_full, full_to_history, glb_iter, staleness_thres)
    return thres



def ring_lookup(full2slot, checkin, ids, now, age_limit, table_f32=None):
    """Lookup of a ring table with the age bound applied at lookup time: the slot of every id, -1
    when the id has no entry or the entry is at least ``age_limit`` iterations old
    (now - checkin[slot] >= age_limit); the reference bounds the age of an entry by un-mapping old
    slots (history_table.py:189-200).  With ``table_f32`` also the rows of the hits (zeros elsewhere)."""
    full2slot, checkin, ids = (np.asarray(a, np.int64) for a in (full2slot, checkin, ids))
    slot = full2slot[ids].copy()
    held = slot >= 0
    stale = held & ((int(now) - checkin[np.maximum(slot, 0)]) >= int(age_limit))
    slot[stale] = -1
    if table_f32 is None:
        return slot
    rows = np.zeros((len(ids), table_f32.shape[1]), np.float32)
    hit = slot >= 0
    rows[hit] = table_f32[slot[hit]]
    return slot, rows
