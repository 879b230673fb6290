"""Zero-copy node-feature store: features stay in pinned host memory and the GPU reads the
requested rows directly over the host link with a gather kernel.

It offers the three members of ``cxgnndl.UVM`` that the cache uses -- ``buffer``, ``get(ids)``,
``masked_get(ids, mask)`` (call sites: /root/reference/hiscache/history_cache.py:161,283,301,345).
``masked_get`` returns zeros for rows whose mask is false: the caller adds cached features on top
(history_cache.py:345-349).

Two tiers: ``set_hot_rows(hot_ids)`` keeps copies of the most requested rows in device memory (the feature half
of the reference's cache: hotness-ordered rows in GPU memory, history_cache.py:121-142); every read then takes
those rows from there and only the others over the host link, with the same result."""
import torch

import hiscache_backend as _be


class PinnedFeatureStore:

    def __init__(self, features, device="cuda:0", out_dtype=torch.float32, prefetch_cus=0, hot_ids=None):
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
        self.hot_rows = None            # [n_hot, F] device copies of the most requested rows, or None
        self.hot_slot = None            # int32 per node: its row in hot_rows, or -1
        self.last_cold = None           # flags of the last tiered read: the rows that came over the host link
        self._inflight = []             # (event, tensors) of reads that may still be running on the read-ahead stream
        if hot_ids is not None:
            self.set_hot_rows(hot_ids)

    def set_hot_rows(self, hot_ids, rows=None, num_nodes=None, chunk_rows=1 << 22):
        """Keep copies of the rows ``hot_ids`` (int64, no duplicates; the head of a hotness order such as
        ``sorted_indices.dat``) in device memory.  ``rows``: the copies, if the caller has them already;
        ``num_nodes``: size of the id space when it is not the number of rows of the host matrix."""
        if self.buffer.is_cuda:
            raise ValueError("the whole matrix is in device memory already")
        hot_ids = torch.as_tensor(hot_ids, dtype=torch.int64).to(self.device).contiguous()
        n_nodes = int(num_nodes if num_nodes is not None else self.buffer.shape[0])
        k = hot_ids.numel()
        if k and (int(hot_ids.min()) < 0 or int(hot_ids.max()) >= n_nodes):
            raise ValueError("hot_ids outside the id space")
        slot = torch.full((n_nodes,), -1, dtype=torch.int32, device=self.device)
        slot[hot_ids] = torch.arange(k, dtype=torch.int32, device=self.device)
        if rows is None:
            rows = torch.empty((k, self.buffer.shape[1]), dtype=self.buffer.dtype, device=self.device)
            for lo in range(0, k, chunk_rows):
                hi = min(k, lo + chunk_rows)
                _be.gather_rows(self.buffer, self._host_ids(hot_ids[lo:hi]), out=rows[lo:hi])
        elif tuple(rows.shape) != (k, self.buffer.shape[1]) or not rows.is_cuda:
            raise ValueError("rows must be a device tensor [len(hot_ids), F]")
        self.hot_rows, self.hot_slot = rows.contiguous(), slot

    def _host_ids(self, ids):
        """Rows of the host matrix that hold the nodes ``ids`` (the ids themselves)."""
        return ids

    def _tiered(self, ids, mask, out, cold_stream):
        """Both tiers' launches: the device tier on the current stream, the host tier on ``cold_stream``."""
        rows, cold = _be.gather_rows_hot(self.hot_rows, self.hot_slot, ids, mask=mask, out=out, out_dtype=self.out_dtype)
        src_ids = self._host_ids(ids)
        if cold_stream is not None:           # (the caller keeps rows, ids and flags alive until that stream is done)
            cold_stream.wait_stream(torch.cuda.current_stream(self.device))
        _be.gather_rows_flagged(self.buffer, src_ids, cold, rows, stream=cold_stream)
        self.last_cold = cold
        return rows, src_ids

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
        makes a new stream.  Reads in flight are waited for; tensors handed out earlier stay valid."""
        side, self._prefetch_side = self._prefetch_side, None
        if side is not None:
            side.synchronize()
            self._inflight.clear()
            if self.prefetch_cus > 0:
                _be.release_cu_limited_stream(side)

    def get(self, ids):
        return self.masked_get(ids, None)

    def masked_get(self, ids, mask):
        if self.hot_rows is not None:
            return self._tiered(ids, mask, None, None)[0]
        return _be.gather_rows(self.buffer, self._host_ids(ids), mask=mask, out_dtype=self.out_dtype)

    def masked_get_async(self, ids, mask):
        """Start the gather on a side stream (default priority) that first waits for the work
        queued so far on the current stream.  Returns (tensor, event); wait on the event (or call
        ``join``) before reading the tensor on another stream."""
        cur = torch.cuda.current_stream(self.device)
        side = self._side_stream()
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            out = self.masked_get(ids, mask)
            self._done.record(side)
        out.record_stream(cur)
        ids.record_stream(side)          # the caller may drop its last reference before the read is done
        mask.record_stream(side)
        return out, self._done

    def join(self, event):
        torch.cuda.current_stream(self.device).wait_event(event)

    def quiet_stream(self, candidates=4, rows=60_000, kernels=24, apart_from=()):
        """A stream (default priority) for the work that runs beside ``prefetch``'s reads, chosen by measurement.
        Which hardware queue a stream shares decides how much a host-link read on the read-ahead stream slows the
        kernels that start beside it: about 2x on most queues, 5 - 30x on an unlucky one (a 0.9 ms iteration then
        takes 2.2 ms), and a program cannot ask which it got.  So ``candidates`` streams are tried in turn: ``kernels``
        small launches are timed on each while ``rows`` random rows are being read, and the one that finishes them
        soonest is returned.  ``apart_from``: streams (the sampler's, say) whose hardware queue the result must not
        share either.  A few milliseconds, once; without a read-ahead stream of limited width only ``apart_from``
        is looked at."""
        apart_from = [torch.cuda.current_stream(self.device)] + list(apart_from)
        if self.prefetch_cus <= 0 or self.buffer.is_cuda:
            return _be.stream_apart_from(apart_from, self.device)
        if self._prefetch_side is None:
            self._prefetch_side = self._make_prefetch_stream()
        side, cur = self._prefetch_side, torch.cuda.current_stream(self.device)
        n = int(self.buffer.shape[0])
        rows = max(1, min(int(rows), n))
        ids = torch.randint(0, n, (rows,), device=self.device)
        out = torch.empty((rows, self.buffer.shape[1]), dtype=self.out_dtype, device=self.device)
        small = torch.zeros(1 << 16, device=self.device)
        best, best_ms = None, None
        for _ in range(max(1, int(candidates))):
            cand = _be.stream_apart_from(apart_from, self.device)
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize(self.device)
            cand.wait_stream(cur)
            side.wait_stream(cur)
            _be.gather_rows(self.buffer, self._host_ids(ids), out=out, stream=side)
            with torch.cuda.stream(cand):
                t0.record()
                for _ in range(int(kernels)):
                    small.add_(1.0)
                t1.record()
            torch.cuda.synchronize(self.device)
            ms = t0.elapsed_time(t1)
            if best_ms is None or ms < best_ms:
                best, best_ms = cand, ms
        self.quiet_stream_ms = best_ms
        return best

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
        if self.hot_rows is not None:
            # the rows with a device copy are taken here and now (a few microseconds at full width); only the
            # others wait for the host link, on the side stream
            rows, src_ids = self._tiered(ids, mask, out, side)
        else:
            src_ids = self._host_ids(ids)
            side.wait_stream(cur)                  # the ids are produced on the current stream
            # enqueued on the side stream by name: switching torch's current stream and back costs the host 20 us
            rows = _be.gather_rows(self.buffer, src_ids, mask=mask, out=out, out_dtype=self.out_dtype, stream=side)
        done = torch.cuda.Event()
        done.record(side)
        # What the read touches stays referenced here until the read has finished, whatever becomes of the handle.
        # (Marking the tensors as used by the side stream -- ``record_stream`` -- would do as well, but then torch's
        # allocator touches that stream whenever one of them is freed, and a stream kept to a few compute units is
        # destroyed by ``close()`` or at interpreter exit, possibly before the last of them.)
        self._inflight = [entry for entry in self._inflight if not entry[0].query()]
        self._inflight.append((done, (rows, ids, src_ids, mask, self.last_cold)))
        handle = PrefetchedRows(ids, rows, done, mask)
        handle.src_ids = src_ids
        return handle

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
