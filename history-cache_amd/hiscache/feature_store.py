"""Zero-copy node-feature store: features stay in pinned host memory and the GPU reads the
requested rows directly over the host link with a gather kernel.

It offers the three members of ``cxgnndl.UVM`` that the cache uses -- ``buffer``, ``get(ids)``,
``masked_get(ids, mask)`` (call sites: /root/reference/hiscache/history_cache.py:161,283,301,345).
``masked_get`` returns zeros for rows whose mask is false: the caller adds cached features on top
(history_cache.py:345-349)."""
import torch

import hiscache_backend as _be


class PinnedFeatureStore:

    def __init__(self, features, device="cuda:0", out_dtype=torch.float32):
        # out_dtype: element type of the gathered rows (keep torch.float16 for fp16 feature files to
        # halve the traffic of the first aggregation layer)
        self.out_dtype = out_dtype
        if features.dim() != 2:
            raise ValueError("features must be [num_nodes, feature_dim]")
        if features.is_cuda:
            self.buffer = features.contiguous()
        else:
            buf = features.contiguous()
            if not buf.is_pinned():
                pinned = torch.empty(buf.shape, dtype=buf.dtype, pin_memory=True)
                pinned.copy_(buf)
                buf = pinned
            self.buffer = buf
        self.device = torch.device(device)
        self._side = None
        self._done = None
        self._prefetch_side = None

    def _side_stream(self):
        if self._side is None:
            self._side = torch.cuda.Stream(device=self.device)
            self._done = torch.cuda.Event()
        return self._side

    def get(self, ids):
        return _be.gather_rows(self.buffer, ids, out_dtype=self.out_dtype)

    def masked_get(self, ids, mask):
        return _be.gather_rows(self.buffer, ids, mask=mask, out_dtype=self.out_dtype)

    def masked_get_async(self, ids, mask):
        """Start the gather on a side stream (default priority) that first waits for the work
        queued so far on the current stream.  Returns (tensor, event); wait on the event (or call
        ``join``) before reading the tensor on another stream."""
        cur = torch.cuda.current_stream(self.device)
        side = self._side_stream()
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            out = _be.gather_rows(self.buffer, ids, mask=mask, out_dtype=self.out_dtype)
            self._done.record(side)
        out.record_stream(cur)
        ids.record_stream(side)          # the caller may drop its last reference before the read is done
        mask.record_stream(side)
        return out, self._done

    def join(self, event):
        torch.cuda.current_stream(self.device).wait_event(event)

    def prefetch(self, ids):
        """Start reading the rows of ALL ``ids`` on a side stream (default priority) now, so that the
        host-link read overlaps whatever the caller queues next -- typically the previous batch's
        forward and backward.  No mask: which rows the cache makes unnecessary is not known before that
        batch's update.  Returns a handle for ``take``."""
        cur = torch.cuda.current_stream(self.device)
        if self._prefetch_side is None:
            self._prefetch_side = torch.cuda.Stream(device=self.device)
        side = self._prefetch_side
        side.wait_stream(cur)                      # the ids are produced on the current stream
        with torch.cuda.stream(side):
            rows = _be.gather_rows(self.buffer, ids, out_dtype=self.out_dtype)
            done = torch.cuda.Event()
            done.record(side)
        ids.record_stream(side)
        return PrefetchedRows(ids, rows, done)

    def take(self, handle):
        """The rows of a ``prefetch``; the current stream waits for the read to finish."""
        cur = torch.cuda.current_stream(self.device)
        cur.wait_event(handle.done)
        handle.rows.record_stream(cur)
        return handle.rows


class PrefetchedRows:
    __slots__ = ("ids", "rows", "done")

    def __init__(self, ids, rows, done):
        self.ids, self.rows, self.done = ids, rows, done
