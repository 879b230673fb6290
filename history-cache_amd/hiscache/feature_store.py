"""Zero-copy node-feature store: features stay in pinned host memory and the GPU reads the
requested rows directly over the host link with a gather kernel.

It offers the three members of ``cxgnndl.UVM`` that the cache uses -- ``buffer``, ``get(ids)``,
``masked_get(ids, mask)`` (call sites: /root/reference/hiscache/history_cache.py:161,283,301,345).
``masked_get`` returns zeros for rows whose mask is false: the caller adds cached features on top
(history_cache.py:345-349)."""
import torch

import hiscache_backend as _be


class PinnedFeatureStore:

    def __init__(self, features, device="cuda:0", out_dtype=torch.float32, prefetch_cus=0):
        # out_dtype: element type of the gathered rows (keep torch.float16 for fp16 feature files to
        # halve the traffic of the first aggregation layer)
        # prefetch_cus > 0: ``prefetch`` reads on a stream that is kept to that many compute units, so that
        # the read, which waits on the host link, does not slow the compute it runs beside (16 - 32 units
        # still saturate the link; the compute must run on a non-default stream for the two to overlap)
        self.out_dtype = out_dtype
        self.prefetch_cus = int(prefetch_cus)
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

    def _make_prefetch_stream(self):
        if self.prefetch_cus > 0:
            return _be.cu_limited_stream(self.prefetch_cus, self.device)
        return torch.cuda.Stream(device=self.device)

    def close(self):
        """Release the read-ahead stream (a CU-limited stream is a driver object that lives until it is
        destroyed; without this it goes at interpreter exit).  The store stays usable: the next ``prefetch``
        makes a new stream."""
        side, self._prefetch_side = self._prefetch_side, None
        if side is not None and self.prefetch_cus > 0:
            _be.release_cu_limited_stream(side)

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

    def prefetch(self, ids, mask=None, out=None):
        """Start reading the rows of ``ids`` (all of them, or those flagged by ``mask``: the caller's guess
        of which will be needed) on a side stream (default priority) now, so that the host-link read
        overlaps whatever the caller queues next -- typically the previous batch's forward and
        backward.  Returns a handle for ``take``; ``handle.mask`` is the mask that was read under.
        ``out`` ([len(ids), F], optional): where the rows go instead of a new tensor."""
        cur = torch.cuda.current_stream(self.device)
        if self._prefetch_side is None:
            self._prefetch_side = self._make_prefetch_stream()
        side = self._prefetch_side
        side.wait_stream(cur)                      # the ids are produced on the current stream
        # enqueued on the side stream by name: switching torch's current stream and back costs the host 20 us
        rows = _be.gather_rows(self.buffer, ids, mask=mask, out=out, out_dtype=self.out_dtype, stream=side)
        done = torch.cuda.Event()
        done.record(side)
        rows.record_stream(side)
        ids.record_stream(side)
        if mask is not None:
            mask.record_stream(side)
        return PrefetchedRows(ids, rows, done, mask)

    def take(self, handle, need=None):
        """The rows of a ``prefetch``; the current stream waits for the read to finish.  ``need`` (the
        exact mask, for a read that was started under a guessed one): rows that have become necessary are
        read now, rows that no longer are get cleared -- the result equals ``masked_get(ids, need)``."""
        cur = torch.cuda.current_stream(self.device)
        cur.wait_event(handle.done)
        handle.rows.record_stream(cur)
        if need is not None and handle.mask is not None:
            _be.fixup_rows(self.buffer, handle.src_ids, need, handle.mask, handle.rows)
        return handle.rows


class PrefetchedRows:
    """``ids``: what the caller asked for (its identity tells the batch apart); ``src_ids``: the rows of
    the store that were read for them."""
    __slots__ = ("ids", "src_ids", "rows", "done", "mask")

    def __init__(self, ids, rows, done, mask=None):
        self.ids, self.src_ids, self.rows, self.done, self.mask = ids, ids, rows, done, mask
