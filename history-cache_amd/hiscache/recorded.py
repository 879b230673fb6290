"""RecordedIteration: one training iteration -- ``lookup_and_load`` -> forward -> loss -> backward ->
optimizer -> ``update_history`` -- recorded once per batch shape in a HIP graph and replayed for every batch.

The loop of the reference (/root/reference/hiscache/history_trainer.py:176-193) enqueues an iteration operator
by operator; for sampled mini-batches of a few thousand rows that is a hundred launches of a few microseconds
each, and the host cannot enqueue them as fast as the GPU runs them.  A recording replays them as one launch.
What stands in the way is that no two sampled batches have the same sizes, so:

* a batch is PADDED into arrays of fixed sizes (one ``hiscache_backend.stage_arrays`` launch): row offsets
  continued at the edge count, node ids at -1.  Padding rows have no edges, aggregate to zero, are never
  referenced by a real row and receive no gradient.  Every layer gets row offsets of its own, flat behind its
  real rows: the rows between a layer's count and the padded one are real rows of the next hop, whose sources
  lie beyond the layer's input, and have to stay empty for that layer;
* the sizes a result depends on are read from device memory, where the same launch writes them: the batch
  normalisation counts only the real rows and gives the others a zero output and a zero gradient, the ring
  lookup reports padding as absent, the admission threshold is the quantile of the real rows' scores,
  padding is never admitted, and lookup and admission take the iteration number from there;
* shapes come from one family: the first batch's sizes scaled by ``step ** j`` and rounded up to
  ``round_to`` rows, the smallest ``j`` that holds the batch.  The sizes of a sampled batch move together, so
  a handful of recordings serve a run; each is made the second time its shape is asked for (the first time the
  same padded iteration runs unrecorded, which also lets the GEMM library settle on its kernels outside a
  recording).

The model is a ``HistorySAGE`` or a ``HistoryRGCN`` in training mode with the fused epilogue, the cache a
``RingHistoryCache`` or a ``HistoryCache`` that admits by gradient, the optimizer one whose step can be recorded
(``capturable=True``).  The cache's hit counters are not kept for recorded iterations.
"""
import math
from types import SimpleNamespace

import torch

import hiscache_backend as _be

from .util import backward_on_this_thread


class _Record:
    __slots__ = ("caps", "e_cap", "batch", "scal", "graph", "loss", "uses", "ptr", "idx", "s2f", "y", "ptrT", "rowT",
                 "edgeT", "etype", "x_pre", "have", "src_ids", "ptrs")


class RecordedIteration:

    def __init__(self, model, cache, optimizer, num_layers, loss_fn=None, step=1.125, round_to=256,
                 max_records=16, with_view=True, record=True, read_ahead_slots=2):
        self.model, self.cache, self.optimizer = model, cache, optimizer
        self.L = int(num_layers)
        self.loss_fn = loss_fn or torch.nn.functional.nll_loss
        self.step = float(step)
        self.round_to = int(round_to)
        self.max_records = int(max_records)
        self.with_view = bool(with_view)
        self.record = bool(record)        # False: the padded iterations run, but none is recorded (for comparison)
        # rows read ahead go straight into a recording's own array; a shape then has this many recordings, used in
        # turn, so that the read for a coming batch never writes what the replay in flight reads (read at most
        # read_ahead_slots - 1 batches ahead)
        self.read_ahead_slots = max(1, int(read_ahead_slots))
        self._reads_started = 0
        self.device = cache.device
        self._hub_edges = _be.bwd_chunk_edges(256) or (1 << 62)
        self._base = None                 # sizes of the first batch: (n0, [n1 .. nL], E)
        self._records = {}
        self._capture_stream = None
        self.replays = 0
        self.unrecorded = 0

    # ------------------------------------------------------------------ shapes
    def _key_for(self, nnl, n_edges):
        if self._base is None:
            self._base = (int(nnl[0]), [max(int(v), 1) for v in nnl[1:]], max(int(n_edges), 1))
        n0, base_n, base_e = self._base
        if int(nnl[0]) != n0:
            return None                    # another number of seeds (the last batch of an epoch): not recorded
        need = max(max(int(v) / b for v, b in zip(nnl[1:], base_n)), int(n_edges) / base_e)
        j = math.ceil(math.log(need) / math.log(self.step) - 1e-9) if need > 0 else 0
        while not self._holds(j, nnl, n_edges):        # rounding of the logarithm
            j += 1
        # the rounding up of the rows may leave room one step below (and below that, while the shape still shrinks)
        while self._shape(j - 1) != self._shape(j) and self._holds(j - 1, nnl, n_edges):
            j -= 1
        return j

    def _shape(self, j):
        n0, base_n, base_e = self._base
        up = lambda v: (int(math.ceil(v * self.step ** j)) + self.round_to - 1) // self.round_to * self.round_to
        caps = [n0] + [up(b) for b in base_n]
        for k in range(1, len(caps)):                  # a layer's rows are a prefix of the next layer's
            caps[k] = max(caps[k], caps[k - 1])
        return caps, up(base_e)

    def _holds(self, j, nnl, n_edges):
        caps, e_cap = self._shape(j)
        return all(int(v) <= c for v, c in zip(nnl, caps)) and int(n_edges) <= e_cap

    def _describe(self, batch):
        nnl = [int(v) for v in batch.num_node_in_layer]
        n_edges = int(batch.idx.numel())
        view = getattr(batch, "view", None) if self.with_view else None
        if view is not None and (view.rows < nnl[self.L - 1] or view.n_src < nnl[self.L]):
            view = None
        view_kind = 0 if view is None else (2 if view.edgeT is not None else 1)
        # a view known to hold no source above the backward's chunk length is recorded without the hub launches
        if view is not None and view.max_in_degree is not None and view.max_in_degree <= self._hub_edges:
            view_kind += 10
        return nnl, n_edges, view_kind, getattr(batch, "edge_type", None)

    # ------------------------------------------------------------------ records
    def _new_record(self, j, view_kind, pre_like, etype):
        L, dev = self.L, self.device
        hubless, view_kind = view_kind >= 10, view_kind % 10
        has_view = view_kind > 0
        caps, e_cap = self._shape(j)
        r = _Record()
        r.caps, r.e_cap, r.graph, r.loss, r.uses = caps, e_cap, None, None, 0
        i64 = dict(dtype=torch.int64, device=dev)
        r.ptr = torch.zeros(caps[L - 1] + 1, **i64)
        # Row offsets of every layer's own: those of the batch up to the layer's real rows, flat behind them.  The
        # rows between a layer's real count and its padded count are real rows of the NEXT hop, whose sources lie
        # beyond the layer's input: with the batch's own offsets the layer would aggregate them, reading behind
        # its input.  (The last entry, the layer that covers every row of the batch, is the batch's array.)
        r.ptrs = [torch.zeros(caps[k] + 1, **i64) for k in range(L - 1)] + [r.ptr]
        r.idx = torch.zeros(e_cap, **i64)
        r.s2f = torch.full((caps[L],), -1, **i64)
        r.y = torch.zeros(caps[0], **i64)
        r.ptrT = torch.zeros(caps[L] + 1, **i64) if has_view else None
        r.rowT = torch.zeros(e_cap, dtype=torch.int32, device=dev) if has_view else None
        r.edgeT = torch.zeros(e_cap, dtype=torch.int32, device=dev) if view_kind == 2 else None
        r.etype = torch.zeros(e_cap, dtype=etype.dtype, device=dev) if etype is not None else None
        r.scal = torch.zeros(L + 4, **i64)             # nnl[0..L], edges, now, it
        r.x_pre = r.have = r.src_ids = None
        pre = None
        if pre_like is not None:                       # feature rows read ahead of time land here: (width, dtype)
            r.x_pre = torch.zeros((caps[L], pre_like[0]), dtype=pre_like[1], device=dev)
            r.have = torch.zeros(caps[L], dtype=torch.uint8, device=dev)
            r.src_ids = torch.full((caps[L],), -1, **i64)
            pre = SimpleNamespace(rows=r.x_pre, have=r.have, src_ids=r.src_ids)
        view = (_be.BatchView(r.ptrT, r.rowT, r.edgeT, caps[L - 1], caps[L], e_cap, 0 if hubless else None)
                if has_view else None)
        r.batch = SimpleNamespace(
            ptr=r.ptr, idx=r.idx, sub_to_full=r.s2f, y=r.y, x=None, edge_type=r.etype, typed_num_node_in_layer=None,
            num_node_in_layer=torch.tensor(caps, dtype=torch.int64), num_edge_in_layer=[e_cap] * L, view=view,
            ptr_of_layer=r.ptrs,
            dev=SimpleNamespace(nnl=[r.scal[k:k + 1] for k in range(L + 1)], edges=r.scal[L + 1:L + 2],
                                now=r.scal[L + 2:L + 3], it=r.scal[L + 3:L + 4],
                                row_index=torch.arange(caps[L], **i64), prefetched=pre))
        return r

    def _stage(self, r, batch, nnl, n_edges, now, it, handle):
        L = self.L
        n_rows, n_all = int(nnl[L - 1]), int(nnl[L])
        arrays = [(batch.ptr, r.ptr, n_rows + 1, n_edges), (batch.idx, r.idx, n_edges, 0),
                  (batch.sub_to_full, r.s2f, n_all, -1), (batch.y, r.y, int(nnl[0]), 0)]
        nel = batch.num_edge_in_layer                  # edges of the first nnl[k] rows
        arrays += [(batch.ptr, r.ptrs[k], int(nnl[k]) + 1, int(nel[k])) for k in range(L - 1)]
        if r.ptrT is not None:
            v = batch.view
            arrays += [(v.ptrT, r.ptrT, n_all + 1, n_edges), (v.rowT, r.rowT, n_edges, 0)]
            if r.edgeT is not None:
                arrays.append((v.edgeT, r.edgeT, n_edges, 0))
        if r.etype is not None:
            arrays.append((batch.edge_type, r.etype, n_edges, -1))
        if handle is not None:
            torch.cuda.current_stream(self.device).wait_event(handle.done)
            if handle.rows.data_ptr() == r.x_pre.data_ptr():       # read straight into this array: clear what lies behind
                if n_all < r.x_pre.shape[0]:
                    arrays.append((None, r.x_pre[n_all:].view(-1), 0, 0))
            else:
                arrays.append((handle.rows.view(-1), r.x_pre.view(-1), n_all * r.x_pre.shape[1], 0))
            arrays += [(handle.mask.view(torch.uint8), r.have, n_all, 0), (handle.src_ids, r.src_ids, n_all, -1)]
            batch.prefetched_x = None
        _be.stage_arrays(arrays, r.scal, [int(v) for v in nnl] + [n_edges, int(now), int(it)])

    def prefetch(self, batch):
        """Start the host-link read of ``batch``'s feature rows now, under the cache's present state, on the
        feature store's read-ahead stream: it then runs beside the iteration that is replayed next, and the
        iteration on ``batch`` reads only the rows that an admission has made necessary since."""
        out = None
        store = self.cache.uvm
        nnl, n_edges, view_kind, etype = self._describe(batch)
        j = self._key_for(nnl, n_edges)
        if j is not None and self.read_ahead_slots > 1 and hasattr(store, "out_dtype") and hasattr(store, "buffer"):
            slot = self._reads_started % self.read_ahead_slots
            self._reads_started += 1
            key = (j, view_kind, slot, etype is not None)
            r = self._records.get(key)
            if r is None and len(self._records) < self.max_records:
                r = self._records[key] = self._new_record(j, view_kind, (store.buffer.shape[1], store.out_dtype), etype)
            if r is not None:
                out = r.x_pre[: nnl[self.L]]
                batch.recorded_key = key
        self.cache.prefetch(batch, speculative=True, num_layer=self.L, out=out)

    def _iteration(self, b):
        self.cache.lookup_and_load(b, self.L)
        out = self.model(b)
        loss = self.loss_fn(out[: b.y.shape[0]], b.y)
        self.optimizer.zero_grad(set_to_none=True)
        backward_on_this_thread(loss)
        self.optimizer.step()
        self.cache.update_history(b, None)
        return loss.detach()

    # ------------------------------------------------------------------ the call
    def __call__(self, batch, glb_iter):
        """Train on ``batch`` (as ``NeighborSampler`` or ``hiscache.synthetic.make_batch`` hand it over);
        ``glb_iter`` is the iteration number the admitted rows are stamped with.  Returns the loss (a device
        tensor that the next call with the same shape overwrites)."""
        nnl, n_edges, view_kind, etype = self._describe(batch)
        handle = getattr(batch, "prefetched_x", None)
        if handle is not None and (handle.ids is not batch.sub_to_full or handle.mask is None
                                   or handle.rows.element_size() not in (4, 2)):
            handle = None
        j = self._key_for(nnl, n_edges)
        # what a cache decides on the host from the iteration number (HistoryCache: has admission started, the
        # periodic restart of its write position) happens here, in front of the replay
        hook = getattr(self.cache, "before_update", None)
        if hook is not None and not hook(glb_iter):
            j = None
        self.cache.glb_iter += 1
        key = None
        if j is not None:
            # slot -1: no rows read ahead; -2: rows read ahead into a tensor of their own (copied in by the staging
            # launch); 0, 1, ..: read straight into the array of that one of the shape's recordings
            key = (j, view_kind, -1 if handle is None else -2, etype is not None)
            own = getattr(batch, "recorded_key", None)
            if handle is not None and own is not None and own[:2] == key[:2] and own in self._records \
                    and self._records[own].x_pre.data_ptr() == handle.rows.data_ptr():
                key = own
        r = None if key is None else self._records.get(key)
        if r is None and key is not None and len(self._records) < self.max_records:
            pre_like = None if handle is None else (handle.rows.shape[1], handle.rows.dtype)
            r = self._records[key] = self._new_record(j, view_kind, pre_like, etype)
        if r is None:
            # a shape outside the family, or more shapes than recordings are kept for: the ordinary iteration
            self.cache.glb_iter -= 1
            self.unrecorded += 1
            b = batch
            self.cache.lookup_and_load(b, self.L)
            out = self.model(b)
            loss = self.loss_fn(out, b.y)
            self.optimizer.zero_grad(set_to_none=True)
            backward_on_this_thread(loss)
            self.optimizer.step()
            self.cache.update_history(b, glb_iter)
            return loss.detach()
        self._stage(r, batch, nnl, n_edges, self.cache.glb_iter, glb_iter, handle)
        r.uses += 1
        if r.uses == 1 or not self.record or _be.CHECK_INPUTS:
            # the same padded iteration, unrecorded (always so under the library's input checks, which synchronise)
            self.unrecorded += 1
            return self._iteration(r.batch)
        if r.graph is None:
            if self._capture_stream is None:
                self._capture_stream = torch.cuda.Stream(device=self.device)    # default priority
                with torch.cuda.stream(self._capture_stream):
                    _be.prepare_stream(self.device)     # per-stream scratch words exist before anything is recorded
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=self._capture_stream):
                r.loss = self._iteration(r.batch)
            r.graph = graph
        r.graph.replay()
        self.replays += 1
        return r.loss

    def clear(self):
        """Drop every recording and its arrays (they are made again on demand)."""
        self._records.clear()

    def shapes(self):
        """The padded shapes in use: {(j, view kind 0/1/2 = none/rows/rows and edge slots -- +10 when the view is known
        to hold no source above the backward's chunk length --, read-ahead slot (-1: no
        rows read ahead, -2: copied in, 0..: read straight into that recording's array), edge types given):
        ([n0 .. nL], edges, recorded?, uses)}."""
        return {k: (r.caps, r.e_cap, r.graph is not None, r.uses) for k, r in self._records.items()}
