"""HistoryCache: one flat GPU buffer holding hot raw features (filled from the end) and
historical embeddings (appended from the front), with the id maps and the admission policy.

Same public surface as the reference class (/root/reference/hiscache/history_cache.py):
``lookup_and_load(batch, num_layer, feature_cache_only=False)``, ``update_history(batch, glb_iter)``
and the attributes the model and trainers read (``sub2embed``, ``cached_embedding``,
``produced_embedding``, ``used_masks``, ``method``, ``buffer``, ``full2embed``, ``embed2full``,
``feat2full``, ``header``, ``glb_iter``).  The hot steps run as gfx950 kernels through
``hiscache_backend``; nothing on the per-iteration path synchronises with the host.

Differences that a caller can see:
  * sizes and the hot-node list may be passed as arguments instead of being read from
    ``processed/num_nodes.txt`` / ``processed/sorted_indices.dat`` (both still work);
  * ``header`` lives on the device; reading the attribute synchronises;
  * rows that would be appended beyond the buffer are dropped and counted in ``overflow``
    (the reference raises a shape error there, history_cache.py:219-221);
  * ``num_layer`` of ``lookup_and_load`` may be omitted (taken from the config);
  * a ``feature_cache_only`` lookup works in the modes without a cache too (all rows from the store), and
    clears ``used_masks`` (the reference leaves the last training batch's masks
    in place, which its relational model then applies to the evaluation batch).
"""
import math
import time
from os import path

import numpy as np
import torch

import hiscache_backend as _be

from .util import log, quantile_threshold


class HistoryCache:

    def __init__(self, uvm, config, mode, device_id=-1, total_num_node=None, buffer_bytes=None,
                 hot_ids=None):
        self.in_channels = config.dl.dataset.feature_dim
        self.out_channels = config.dl.dataset.num_classes
        self.hidden_channels = config.train.model.hidden_dim
        self.num_layers_all = config.train.model.num_layers
        if total_num_node is None:
            total_num_node = int(
                open(path.join(str(config["dl"]["dataset"]["path"]), "processed",
                               "num_nodes.txt")).readline())
        self.total_num_node = int(total_num_node)
        self.num_device = 1
        self.device_id = device_id
        self.start_history = config.history.start_history
        if config["dl"]["num_device"] > 1:
            raise NotImplementedError("one GPU per cache; the multi-GPU trainer is out of scope")
        self.device = torch.device(config["dl"]["device"])
        self.method = config.history["method"]
        self.rate = float(config.history["rate"])
        assert self.method in ["random", "grad", "staleness"]
        self.staleness_thres = int(config.history.staleness_thres)
        self.limit = float(config.history.limit)

        self.full2embed = torch.full((self.total_num_node * 2 + 1,), -1, dtype=torch.int64,
                                     device=self.device)
        self._header = torch.zeros(1, dtype=torch.int64, device=self.device)
        self._overflow = torch.zeros(1, dtype=torch.int64, device=self.device)
        # what the lookups find (hiscache_backend.STAT_NAMES), counted on the device and read by stats() only
        self._counters = torch.zeros(8, dtype=torch.int64, device=self.device)
        self._uncounted_mask = None
        self._num_stored = torch.zeros(1, dtype=torch.int64, device=self.device)
        self.produced_embedding = None
        self.feat_mode = mode
        self.uvm = uvm
        self.glb_iter = 0
        self.used_masks = None
        self.sub2embed = None
        self.sub2feat = None
        self.cached_embedding = None
        self.last_record_mask = None
        self.distributed_store = False
        self.feat2full = torch.empty(0, dtype=torch.int64, device=self.device)
        if "history" in self.feat_mode:
            self.allocate(buffer_bytes)
            self.fill(config, hot_ids)

    # ------------------------------------------------------------------ attributes kept on device
    @property
    def header(self):
        return int(self._header.item())

    @header.setter
    def header(self, v):
        self._header.fill_(int(v))

    @property
    def overflow(self):
        return int(self._overflow.item())

    @property
    def num_stored_history(self):
        return int(self._num_stored.item())

    # ------------------------------------------------------------------ sizing and pre-fill
    def allocate(self, buffer_bytes=None):
        """Size the flat buffer (/root/reference/hiscache/history_cache.py:95-119): free device
        memory minus 4 GiB, capped by ``limit`` GiB, rounded up to a multiple of
        lcm(hidden, in_channels) floats.  ``buffer_bytes`` overrides the free-memory probe."""
        t0 = time.time()
        if buffer_bytes is None:
            max_byte = torch.cuda.mem_get_info(self.device)[0] - 4 * 1024 * 1024 * 1024
        else:
            max_byte = int(buffer_bytes)
        lcm = self.hidden_channels * self.in_channels // math.gcd(self.hidden_channels,
                                                                  self.in_channels)
        max_buffer_byte = max_byte
        if self.limit > 0 and max_buffer_byte > self.limit * 1024 * 1024 * 1024:
            max_buffer_byte = int(self.limit * 1024 * 1024 * 1024)
        max_buffer_byte = (max_buffer_byte + 4 * lcm - 1) // (4 * lcm) * (4 * lcm)
        n_float = max_buffer_byte // 4
        self.buffer = torch.empty([n_float], dtype=torch.float32, device=self.device)
        self.embed2full = torch.full((n_float // self.hidden_channels,), -1, dtype=torch.int64,
                                     device=self.device)
        self.overall_feat_num = n_float // self.in_channels
        self.overall_embed_num = n_float // self.hidden_channels
        self.max_buffer_byte = max_buffer_byte
        log.info(f"allocating buffer of {n_float} floats: {time.time() - t0:.3f}s")

    def fill(self, config, hot_ids=None):
        """Pre-fill the tail of the buffer with the raw features of the hottest nodes
        (/root/reference/hiscache/history_cache.py:121-178).  ``hot_ids`` (int64, hottest last)
        replaces ``processed/sorted_indices.dat``."""
        t0 = time.time()
        if hot_ids is None:
            p = path.join(str(config["dl"]["dataset"]["path"]), "processed", "sorted_indices.dat")
            indice = torch.from_numpy(np.fromfile(p, dtype=np.int64))
        else:
            indice = torch.as_tensor(hot_ids, dtype=torch.int64).cpu()
        if self.overall_feat_num > self.total_num_node:
            cache_indice = indice
        else:
            cache_indice = indice[-self.overall_feat_num:] if self.overall_feat_num > 0 else indice[:0]
        n_cached = cache_indice.shape[0]
        # Feature slot i of the buffer (viewed as [overall_feat_num, in_channels]) holds node
        # feat2full[i] - total_num_node; the cached block sits at the end of the view and empty
        # slots hold -1.  (The reference keeps only the cached block in feat2full, which shifts
        # its slot arithmetic when the buffer could hold more than all features,
        # history_cache.py:136-137 against :223-226.)
        first = self.overall_feat_num - n_cached
        new_id = torch.arange(first, first + n_cached, device=self.device)
        self.feat2full = torch.full((self.overall_feat_num,), -1, dtype=torch.int64,
                                    device=self.device)
        cached_full = cache_indice.to(self.device) + self.total_num_node
        self.feat2full[first:] = cached_full
        self.full2embed[cached_full] = new_id
        if n_cached > 0:
            rows = _be.gather_rows(self.uvm.buffer, cache_indice.to(self.device))
            self.buffer.view(-1, self.in_channels)[first:self.overall_feat_num] = rows
        log.info(f"filling buffer with {n_cached} raw feature rows: {time.time() - t0:.3f}s")

    # ------------------------------------------------------------------ admission
    @torch.no_grad()
    def update_history(self, batch, glb_iter):
        """Gradient-based admission (/root/reference/hiscache/history_cache.py:180-255):
        score = ||dL/d embedding||_2 per row, thres = quantile(score, rate), rows with
        score < thres that are not cached are appended at ``header``; overlapped feature slots
        and overwritten embedding slots are invalidated; maps and header advance."""
        if "history" not in self.feat_mode or self.staleness_thres == 0:
            return
        # A batch padded to fixed sizes for a recorded iteration (hiscache.RecordedIteration) carries its real
        # sizes on the device; what depends on the iteration number on the HOST -- whether admission has started,
        # the periodic restart of the write position -- is then done by ``before_update``, outside the recording.
        dev = getattr(batch, "dev", None)
        if dev is None:
            if glb_iter < self.start_history:
                return
            self._restart_if_due(glb_iter)
        if self.produced_embedding is None:
            raise AssertionError("produced embedding is None")
        emb = self.produced_embedding
        num_node = emb.shape[0]
        # the reference asserts the same against num_node_in_layer[1] (history_cache.py:200-204): an embedding
        # produced by another layer must not reach the admission kernels
        n1 = int(batch.num_node_in_layer[1])
        if num_node != n1 or self.sub2embed is None or self.sub2embed.numel() < num_node:
            raise ValueError("produced_embedding has {} rows, the batch has {} 1-hop nodes".format(num_node, n1))
        if emb.grad is not None and self.method == "grad":
            g = emb.grad
            assert g.shape[0] == num_node, "grad shape: {}, num_node: {}".format(g.shape, num_node)
            score = _be.row_scores(g.contiguous(), _be.NORM_L2)
        else:
            score = torch.randn([num_node], device=self.device)
        emb.grad = None
        if dev is None:
            thres = quantile_threshold(score, self.rate)
        else:
            # the threshold is the quantile of the real rows' scores; a padding row never passes it
            thres = _be.quantile_select_dev(score, dev.nnl[1], self.rate)
            score = torch.where(dev.row_index[:num_node] < dev.nnl[1], score, torch.full_like(score, float("inf")))
        mask = _be.cache_append(score, thres, emb.detach().contiguous(), self.sub2embed,
                                batch.sub_to_full[:num_node].contiguous(), self.buffer,
                                self.hidden_channels, self.in_channels, self.full2embed,
                                self.embed2full, self.feat2full, self._header, self._overflow)
        self.last_record_mask = mask
        self._uncounted_mask = mask if dev is None else None
        self.last_score = score
        self.produced_embedding = None

    def _restart_if_due(self, glb_iter):
        """Every ``staleness_thres`` iterations the write position goes back to the start of the buffer
        (/root/reference/hiscache/history_cache.py:190-198)."""
        if (glb_iter % self.staleness_thres) == 0:
            torch.maximum(self._num_stored, self._header, out=self._num_stored)
            self._header.zero_()

    def before_update(self, glb_iter):
        """For recorded iterations: the part of ``update_history`` that the host decides from the iteration number,
        run in front of the replay (the lookup does not read the write position, so the order does not matter).
        False when admission has not started yet at ``glb_iter``: that iteration is not one to replay."""
        if "history" not in self.feat_mode or self.staleness_thres == 0:
            return True
        if glb_iter < self.start_history:
            return False
        self._restart_if_due(glb_iter)
        return True

    # ------------------------------------------------------------------ lookup
    def lookup_and_load(self, batch, num_layer=None, feature_cache_only=False):
        """Translate the batch's node ids to cache slots, gather cached embeddings, compute which
        nodes are still needed, load their raw features (zero-copy from host memory, merged with
        the feature cache) into ``batch.x``
        (/root/reference/hiscache/history_cache.py:275-356)."""
        if num_layer is None:
            num_layer = self.num_layers_all
        sub_to_full = batch.sub_to_full
        if feature_cache_only and "history" not in self.feat_mode:
            # no cache was allocated in this mode: every row comes from the store (the reference reads its
            # missing buffer here, /root/reference/hiscache/history_cache.py:276-288)
            batch.x = self.uvm.get(sub_to_full)
            self.used_masks = None
            return None
        if feature_cache_only:
            self.sub2feat = _be.lookup(self.full2embed, sub_to_full, self.total_num_node)
            hit = self.sub2feat != -1
            x = self.uvm.masked_get(sub_to_full, ~hit)
            # the feature cache's rows go where the store left zeros (the reference adds them on top, :285-287)
            _be.gather_rows_flagged(self.buffer.view(-1, self.in_channels), self.sub2feat, hit, x)
            batch.x = x
            self.used_masks = None          # nothing is pruned in evaluation: no masks of an earlier batch linger
            return None

        n1 = int(batch.num_node_in_layer[1])
        if "history" not in self.feat_mode:
            self.sub2embed = torch.full((n1,), -1, dtype=torch.int64, device=self.device)
            self.cached_embedding = torch.empty(0, device=self.device)
            if self.feat_mode in ["uvm", "mmap"]:
                batch.x = self.uvm.get(sub_to_full)
            else:
                raise AssertionError("unsupported feat_mode " + str(self.feat_mode))
            return None

        layer1_nodes = sub_to_full[:n1]
        dev = getattr(batch, "dev", None)
        # a padded batch (recorded iterations): the rows behind the real 1-hop nodes are real nodes of the next
        # hop or padding, and count as not cached; so do the padding nodes for the feature cache
        self.sub2embed = _be.lookup(self.full2embed, layer1_nodes, 0, n_valid=None if dev is None else dev.nnl[1])
        self.sub2feat = _be.lookup(self.full2embed, sub_to_full, self.total_num_node,
                                   n_valid=None if dev is None else dev.nnl[-1])
        self.used_masks = _be.count_history_reconstruct(batch.ptr, batch.idx, self.sub2embed,
                                                        sub_to_full.shape[0], batch.y.shape[0],
                                                        num_layer)
        # hit_feat = sub2feat != -1, load = used & ~hit_feat (reference :327-330) and the hit counters, one launch
        # (the counters are not kept for recorded iterations)
        hit_feat_mask, load_mask = _be.load_mask(self.used_masks[0], self.sub2feat, self.sub2embed,
                                                 self._counted_mask() if dev is None else None,
                                                 self._counters if dev is None else None)
        if dev is None:
            self.glb_iter += 1
        if dev is not None and getattr(dev, "prefetched", None) is not None:
            # rows read ahead of time into the recording's own arrays, under the masks of an earlier cache state
            p = dev.prefetched
            _be.fixup_rows(self.uvm.buffer, p.src_ids, load_mask, p.have, p.rows)
            pre, exact = p.rows, True
        else:
            pre, exact = self._take_prefetched(batch, load_mask)
        if pre is not None and not exact:
            # every row was read ahead of time: keep what masked_get + the feature-cache merge would have
            # produced (needed rows and feature-cache hits), zero the rest
            self.cached_embedding = _be.gather_rows(self.buffer.view(-1, self.hidden_channels),
                                                    self.sub2embed)
            keep = torch.logical_or(self.used_masks[0], hit_feat_mask)
            pre.masked_fill_(~keep[:, None], 0)
            batch.x = pre
            self.load_mask = load_mask
            return None
        # Host-link read of the needed rows.  (Reading it on a side stream here would only overlap
        # the small gather below and costs the host more than that saves; ``prefetch`` is the way to
        # overlap the read with compute.)
        # (a read-ahead under the masks of an earlier cache state was brought to ``load_mask`` when it was taken)
        x = pre if pre is not None else self.uvm.masked_get(sub_to_full, load_mask)
        # slot -1 reads the last row of the view, as the reference's indexing does; such rows
        # are ignored by the aggregation
        self.cached_embedding = _be.gather_rows(self.buffer.view(-1, self.hidden_channels),
                                                self.sub2embed)
        # the feature cache's rows go where the read left zeros (the reference adds them on top, :347-349): only
        # the hit rows are touched
        _be.gather_rows_flagged(self.buffer.view(-1, self.in_channels), self.sub2feat, hit_feat_mask, x)
        batch.x = x
        self.load_mask = load_mask
        return None

    def prefetch(self, batch, speculative=True, num_layer=None, out=None):
        """Start the host-link read of ``batch``'s feature rows now, to overlap it with the work queued
        before that batch's ``lookup_and_load``.  ``speculative``: the rows that the cache's PRESENT state
        makes necessary (slots, used masks and feature-cache hits as ``lookup_and_load`` computes them, one
        update early); ``lookup_and_load`` then reads the rows that have become necessary since and clears
        those that no longer are.  Otherwise every row is read and masked later.  Optional: without it
        ``lookup_and_load`` reads the needed rows itself.  ``batch.x`` comes out the same."""
        start = getattr(self.uvm, "prefetch", None)
        if start is None or "history" not in self.feat_mode:
            return
        if not speculative:
            batch.prefetched_x = start(batch.sub_to_full)
            return
        if num_layer is None:
            num_layer = self.num_layers_all
        sub_to_full = batch.sub_to_full
        n1 = int(batch.num_node_in_layer[1])
        sub2embed = _be.lookup(self.full2embed, sub_to_full[:n1], 0)
        sub2feat = _be.lookup(self.full2embed, sub_to_full, self.total_num_node)
        used = _be.count_history_reconstruct(batch.ptr, batch.idx, sub2embed, sub_to_full.shape[0],
                                             batch.y.shape[0], num_layer)
        _, mask = _be.load_mask(used[0], sub2feat)          # used & (sub2feat == -1), one launch
        # ``out`` (recorded iterations): the rows go straight into the array the recording reads them from
        batch.prefetched_x = start(sub_to_full, mask) if out is None else start(sub_to_full, mask, out=out)

    def _take_prefetched(self, batch, need):
        """(rows, exact): the rows of a read-ahead of this batch, or (None, False).  ``exact``: they were
        read under a mask and have been brought to ``need``, i.e. they equal ``masked_get(ids, need)``."""
        handle = getattr(batch, "prefetched_x", None)
        if handle is None or handle.ids is not batch.sub_to_full:
            return None, False
        batch.prefetched_x = None
        if handle.mask is None:
            return self.uvm.take(handle), False
        return self.uvm.take(handle, need), True

    def _counted_mask(self):
        """The last admission mask, once: the next lookup's launch adds its rows to the counters."""
        m, self._uncounted_mask = self._uncounted_mask, None
        return m

    _STATE = ("buffer", "full2embed", "embed2full", "feat2full", "_header", "_num_stored", "_overflow")

    def state_dict(self):
        """The cache's contents for a checkpoint (the reference saves none): copies of the buffer, the maps and the
        write position, and the iteration counter."""
        if "history" not in self.feat_mode:
            return {"glb_iter": self.glb_iter}
        out = {name.lstrip("_"): getattr(self, name).detach().clone() for name in self._STATE}
        out["glb_iter"] = self.glb_iter
        return out

    def load_state_dict(self, state):
        """Restore what ``state_dict`` saved into a cache of the same sizes."""
        self.glb_iter = int(state["glb_iter"])
        if "history" not in self.feat_mode:
            return
        for name in self._STATE:
            src, dst = state[name.lstrip("_")], getattr(self, name)
            if tuple(src.shape) != tuple(dst.shape) or src.dtype != dst.dtype:
                raise ValueError(f"{name.lstrip('_')}: saved {tuple(src.shape)} {src.dtype}, "
                                 f"this cache has {tuple(dst.shape)} {dst.dtype}")
        for name in self._STATE:
            getattr(self, name).copy_(state[name.lstrip("_")])
        self.produced_embedding = self.sub2embed = self.sub2feat = self.cached_embedding = self.used_masks = None

    def stats(self):
        """Cache occupancy, and what the lookups since construction (or ``reset_stats``) found: hit rates of the
        embedding and the feature cache, rows pruned, rows and bytes read from the feature store, rows admitted
        (the counts that the reference can log from its lookup, hiscache/history_cache.py:331-341).  The counters
        live on the device and are read here only: this call synchronises, the lookups do not."""
        n = self.total_num_node
        c = dict(zip(_be.STAT_NAMES, (int(v) for v in self._counters.tolist())))
        if self._uncounted_mask is not None:             # an update that no lookup has followed yet
            c["rows_admitted"] += int(self._uncounted_mask.sum().item())
        row_bytes = self.in_channels * self.uvm.buffer.element_size() if hasattr(self.uvm, "buffer") else 0
        out = {
            "header": self.header,
            "overflow": self.overflow,
            "embed_cached": int((self.full2embed[:n] != -1).sum().item()),
            "feat_cached": int((self.full2embed[n:2 * n] != -1).sum().item()),
            "glb_iter": self.glb_iter,
        }
        out.update(c)
        out["embedding_hit_rate"] = c["embedding_hits"] / max(c["one_hop_nodes"], 1)
        out["feature_hit_rate"] = c["feature_hits"] / max(c["nodes"], 1)
        out["rows_not_loaded_rate"] = 1.0 - c["rows_loaded"] / max(c["nodes"], 1)    # the reference's "hit-rate"
        out["bytes_from_feature_store"] = c["rows_loaded"] * row_bytes
        return out

    def reset_stats(self):
        self._counters.zero_()
        self._uncounted_mask = None
