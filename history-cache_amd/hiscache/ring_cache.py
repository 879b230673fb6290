"""RingHistoryCache: historical-embedding cache as one ring table in fp32 / fp16 / bf16 with the
admission pass fused on the device.

A build extension for the large synthetic configurations (a 111M x 256 fp16 table does not fit the
reference's flat fp32 buffer design).  It plays the role of ``HistoryCache`` for the model
(/root/reference/hiscache/history_model.py:123-134 reads ``sub2embed``, ``cached_embedding``,
``method`` and sets ``produced_embedding``) and keeps its two entry points,
``lookup_and_load(batch, num_layer)`` and ``update_history(batch, glb_iter)``.  The policy is the
ring of ``HistoryTable`` (/root/reference/hiscache/history_table.py:127-200, kernel
/root/reference/src/cpp/src/grad_check.cu:6-46): a row is admitted when its gradient norm is below
the threshold and it is either not cached or its entry is at least ``age_limit`` iterations old;
admitted rows overwrite the ring in row order.  Norms, test, mask, slot assignment, the
fp32 -> table-dtype row copy and the map updates are one ``hiscache_backend.grad_check`` call.

The age bound is applied at LOOKUP: an entry that is ``age_limit`` iterations old is reported as
absent, so the model recomputes that row from its neighbours and the admission pass may then store
the fresh value (the reference un-maps old slots for the same effect,
/root/reference/hiscache/history_table.py:189-200).  A row that was served from the table is never
re-admitted: what it would store is the cached value itself.
"""
import torch

import hiscache_backend as _be

from .util import quantile_threshold


class RingHistoryCache:

    def __init__(self, uvm, total_num_node, in_channels, hidden_channels, capacity, num_layers,
                 table_dtype=torch.float16, rate=0.5, thres=None, age_limit=1 << 30, method="grad",
                 device="cuda:0", collect_stats=True):
        self.uvm = uvm
        self.total_num_node = int(total_num_node)
        self.in_channels = in_channels
        self.hidden_channels = hidden_channels
        self.num_layers_all = num_layers
        self.device = torch.device(device)
        self.method = method
        self.rate = rate
        self.age_limit = int(age_limit)
        self.table = torch.zeros((capacity, hidden_channels), dtype=table_dtype, device=self.device)
        self.full2slot = torch.full((self.total_num_node,), -1, dtype=torch.int64, device=self.device)
        self.slot2full = torch.full((capacity,), -1, dtype=torch.int64, device=self.device)
        self.checkin = torch.full((capacity,), -1, dtype=torch.int64, device=self.device)
        self._header = torch.zeros(1, dtype=torch.int64, device=self.device)
        # a fixed threshold (1-element tensor) skips the quantile; otherwise quantile(score, rate)
        self.thres = None if thres is None else torch.tensor([float(thres)], dtype=torch.float32,
                                                             device=self.device)
        self.glb_iter = 0
        self.produced_embedding = None
        self.sub2embed = None
        self.cached_embedding = None
        self.used_masks = None
        self.last_record_mask = None
        # what the lookups find (hiscache_backend.STAT_NAMES), counted on the device by one small launch per
        # lookup and read by stats() only; collect_stats=False leaves the launch out
        self._counters = torch.zeros(8, dtype=torch.int64, device=self.device) if collect_stats else None
        self._uncounted_mask = None

    @property
    def header(self):
        return int(self._header.item())

    def lookup_and_load(self, batch, num_layer=None, feature_cache_only=False):
        if num_layer is None:
            num_layer = self.num_layers_all
        sub_to_full = batch.sub_to_full
        if feature_cache_only:
            # evaluation (/root/reference/hiscache/history_cache.py:276-288): every node's features, no embedding
            # is looked up and the table's state is left alone
            batch.x = self.uvm.get(sub_to_full)
            self.sub2embed = self.cached_embedding = self.used_masks = None
            return None
        n1 = int(batch.num_node_in_layer[1])
        # A batch padded to fixed sizes for a recorded iteration (hiscache.RecordedIteration) carries its real
        # sizes and the iteration number on the device: rows behind the real 1-hop nodes find nothing, and this
        # object's own counter is kept by whoever replays the recording.
        dev = getattr(batch, "dev", None)
        if dev is None:
            self.glb_iter += 1
        # slots (stale entries count as absent) and the cached rows of the hits, one launch
        self.sub2embed, self.cached_embedding = _be.ring_lookup(
            self.full2slot, sub_to_full[:n1], self.table, checkin=self.checkin,
            now=self.glb_iter if dev is None else dev.now, age_limit=self.age_limit,
            n_valid=None if dev is None else dev.nnl[1])
        self.used_masks = _be.count_history_reconstruct(batch.ptr, batch.idx, self.sub2embed,
                                                        sub_to_full.shape[0], batch.y.shape[0], num_layer)
        if self._counters is not None and dev is None:
            prev, self._uncounted_mask = self._uncounted_mask, None
            _be.load_mask(self.used_masks[0], None, self.sub2embed, prev, self._counters)
        if dev is not None and getattr(dev, "prefetched", None) is not None:
            # a padded batch whose rows were read ahead of time into fixed arrays (rows, the mask they were read
            # under, the store's row ids): the rows that have become necessary since are read now, those that no
            # longer are get cleared
            pre = dev.prefetched
            _be.fixup_rows(self.uvm.buffer, pre.src_ids, self.used_masks[0], pre.have, pre.rows)
            batch.x = pre.rows
            return None
        handle = getattr(batch, "prefetched_x", None)
        if handle is not None and handle.ids is sub_to_full:
            batch.prefetched_x = None
            if handle.mask is None:
                # every row was read ahead of time: zero the rows the cache makes unnecessary
                x = self.uvm.take(handle)
                x.masked_fill_(~self.used_masks[0][:, None], 0)
            else:
                # the rows were read under the masks of an earlier cache state: the few that have become
                # necessary since are read now, the few that no longer are get cleared
                x = self.uvm.take(handle, self.used_masks[0])
            batch.x = x
            return None
        batch.x = self.uvm.masked_get(sub_to_full, self.used_masks[0])
        return None

    def prefetch(self, batch, speculative=True, num_layer=None, out=None):
        """Start the host-link read of ``batch``'s feature rows now, to overlap it with the work queued
        before that batch's ``lookup_and_load``.  ``speculative``: only the rows that the cache's PRESENT
        state makes necessary are read (a lookup and the used masks, as ``lookup_and_load`` computes
        them, one admission pass early); ``lookup_and_load`` then reads the rows that an admission or an
        overwritten slot has made necessary since and clears those that have become unnecessary, so that
        ``batch.x`` is the same tensor either way.  Otherwise every row is read and masked later."""
        start = getattr(self.uvm, "prefetch", None)
        if start is None:
            return
        if not speculative:
            batch.prefetched_x = start(batch.sub_to_full)
            return
        if num_layer is None:
            num_layer = self.num_layers_all
        sub_to_full = batch.sub_to_full
        n1 = int(batch.num_node_in_layer[1])
        slot, _ = _be.ring_lookup(self.full2slot, sub_to_full[:n1], self.table, checkin=self.checkin,
                                  now=self.glb_iter + 1, age_limit=self.age_limit, want_rows=False)
        masks = _be.count_history_reconstruct(batch.ptr, batch.idx, slot, sub_to_full.shape[0],
                                              batch.y.shape[0], num_layer)
        # ``out`` (recorded iterations): the rows go straight into the array the recording reads them from
        batch.prefetched_x = start(sub_to_full, masks[0]) if out is None else start(sub_to_full, masks[0], out=out)

    @torch.no_grad()
    def update_history(self, batch, glb_iter):
        emb = self.produced_embedding
        if emb is None:
            raise AssertionError("produced embedding is None")
        n1 = emb.shape[0]
        slot = self.sub2embed
        if slot is None or slot.numel() != n1:
            raise ValueError("produced_embedding has %d rows but the last lookup covered %d 1-hop nodes"
                             % (n1, -1 if slot is None else slot.numel()))
        sub_to_full = batch.sub_to_full[:n1].contiguous()
        # rows with a slot were served from the table (stale entries were reported absent at lookup):
        # only rows that were computed in this iteration can be admitted, so no age is passed
        common = dict(checkin=self.checkin)
        dev = getattr(batch, "dev", None)
        if dev is not None:
            # a padded batch: the rows behind the real 1-hop nodes are never admitted, the threshold is the
            # quantile of the real rows' scores, and the iteration number comes from the device
            if self.method != "grad" or emb.grad is None:
                raise ValueError("recorded iterations admit by gradient")
            common["used"] = dev.row_index[:n1] < dev.nnl[1]
            glb_iter = dev.it
        if self.method == "grad" and emb.grad is not None:
            grad = emb.grad.contiguous()
            if self.thres is not None:
                mask, score = _be.grad_check(grad, emb.detach().contiguous(), slot, sub_to_full, self.thres,
                                             self.table, self.full2slot, self.slot2full, self._header, glb_iter,
                                             **common)
            else:
                score = _be.row_scores(grad)
                thres = (quantile_threshold(score, self.rate) if dev is None
                         else _be.quantile_select_dev(score, dev.nnl[1], self.rate))
                mask, _ = _be.grad_check(None, emb.detach().contiguous(), slot, sub_to_full, thres, self.table,
                                         self.full2slot, self.slot2full, self._header, glb_iter, score=score,
                                         **common)
        else:
            score = torch.randn([n1], device=self.device)
            thres = quantile_threshold(score, self.rate)
            mask, _ = _be.grad_check(None, emb.detach().contiguous(), slot, sub_to_full, thres, self.table,
                                     self.full2slot, self.slot2full, self._header, glb_iter, score=score,
                                     **common)
        emb.grad = None
        self.last_record_mask = mask
        self._uncounted_mask = mask if self._counters is not None and dev is None else None
        self.last_score = score
        self.produced_embedding = None

    _STATE = ("table", "full2slot", "slot2full", "checkin", "_header")

    def state_dict(self):
        """The table, its maps and write position and the iteration counter, copied, for a checkpoint."""
        out = {name.lstrip("_"): getattr(self, name).detach().clone() for name in self._STATE}
        out["glb_iter"] = self.glb_iter
        return out

    def load_state_dict(self, state):
        """Restore what ``state_dict`` saved into a cache of the same sizes."""
        for name in self._STATE:
            src, dst = state[name.lstrip("_")], getattr(self, name)
            if tuple(src.shape) != tuple(dst.shape) or src.dtype != dst.dtype:
                raise ValueError(f"{name.lstrip('_')}: saved {tuple(src.shape)} {src.dtype}, "
                                 f"this cache has {tuple(dst.shape)} {dst.dtype}")
        for name in self._STATE:
            getattr(self, name).copy_(state[name.lstrip("_")])
        self.glb_iter = int(state["glb_iter"])
        self.produced_embedding = self.sub2embed = self.cached_embedding = self.used_masks = None

    def stats(self):
        """Table occupancy and what the lookups since construction found: embedding hit rate, rows pruned, rows
        and bytes read from the feature store, rows admitted (the counts of the reference's lookup log,
        /root/reference/hiscache/history_cache.py:331-341).  Synchronises; the lookups do not."""
        out = {"header": self.header, "glb_iter": self.glb_iter,
               "embed_cached": int((self.full2slot != -1).sum().item())}
        if self._counters is None:
            return out
        c = dict(zip(_be.STAT_NAMES, (int(v) for v in self._counters.tolist())))
        if self._uncounted_mask is not None:
            c["rows_admitted"] += int(self._uncounted_mask.sum().item())
        row_bytes = self.in_channels * self.uvm.buffer.element_size() if hasattr(self.uvm, "buffer") else 0
        out.update(c)
        out["embedding_hit_rate"] = c["embedding_hits"] / max(c["one_hop_nodes"], 1)
        out["rows_not_loaded_rate"] = 1.0 - c["rows_loaded"] / max(c["nodes"], 1)
        out["bytes_from_feature_store"] = c["rows_loaded"] * row_bytes
        return out

    def preload(self, node_ids, rows=None):
        """Mark ``node_ids`` (unique int64 on the device) as cached in slots header.. (benchmark /
        warm-start helper).  ``rows`` [len, hidden] fills the table rows, else they stay as they are."""
        n = node_ids.numel()
        h = self.header
        cap = self.table.shape[0]
        if h + n > cap:
            raise ValueError("preload does not wrap the ring")
        slots = torch.arange(h, h + n, device=self.device)
        self.full2slot[node_ids] = slots
        self.slot2full[h:h + n] = node_ids
        self.checkin[h:h + n] = 0
        if rows is not None:
            self.table[h:h + n] = rows.to(self.table.dtype)
        self._header.fill_((h + n) % cap)
