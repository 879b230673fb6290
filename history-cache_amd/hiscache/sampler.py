"""NeighborSampler: layered neighbour sampling on the GPU, producing the batch object the cache and
the model read.

The reference takes its batches from the external ``cxgnndl`` loader
(/root/reference/hiscache/history_trainer.py:19,26); the fields it reads from a batch are ``ptr``,
``idx``, ``sub_to_full``, ``num_node_in_layer``, ``num_edge_in_layer``, ``x`` and ``y``
(/root/reference/hiscache/history_model.py:120-153, history_cache.py:307-324).  This class fills
them from a CSR graph resident in device memory with one library call per batch and one small
device-to-host copy (the layer sizes, which the model needs as Python ints).
"""
from types import SimpleNamespace

import torch

import hiscache_backend as _be


class NeighborSampler:

    def __init__(self, indptr, indices, fanout, labels=None, seed=0, device="cuda:0", validate=True,
                 emit_view=False, view_edges=False, replay_slots=0):
        """``indptr`` / ``indices``: CSR of the full graph (int64; moved to ``device``).  ``fanout[k]``
        neighbours are drawn, without replacement, for nodes first reached at hop k.  ``emit_view``:
        every batch also carries ``batch.view``, the transposed view of its CSR
        (``hiscache_backend.BatchView``), built right behind the sampling on the sampler's stream, so
        that the layers' backward builds none; ``view_edges`` adds the view's edge slots, which the
        relational layer's backward reads.  (The view is built with the batch's sizes still on the device,
        for batches whose capacity -- seeds x the fanouts' products -- stays below 2^24 edges and nodes;
        beyond that the sampling call raises and the batch must come without a view.)
        ``replay_slots`` = K > 0: the launches of one batch (about forty: every one has the same shape for
        the same number of seeds, the sizes stay on the device) are recorded once per slot in a HIP graph and
        replayed as one launch per batch; the batch's arrays then live in the slot's own memory and are
        OVERWRITTEN when the slot comes round again, K batches later -- choose K above the number of batches
        that are alive at once (in flight, being trained on, kept).  Batches with another number of seeds
        (the last one of an epoch) take the ordinary path."""
        self.replay_slots = int(replay_slots)
        self._slots = [None] * self.replay_slots
        self._next_slot = 0
        self.emit_view = bool(emit_view)
        self.view_edges = bool(view_edges)
        self.device = torch.device(device)
        self.indptr = torch.as_tensor(indptr, dtype=torch.int64).to(self.device).contiguous()
        self.indices = torch.as_tensor(indices, dtype=torch.int64).to(self.device).contiguous()
        self.num_nodes = self.indptr.numel() - 1
        self.fanout = [int(f) for f in fanout]
        self.labels = None if labels is None else torch.as_tensor(labels).to(self.device)
        self.seed = int(seed)
        self.batches = 0
        if validate and self.indices.numel():
            lo, hi = int(self.indices.min()), int(self.indices.max())
            if lo < 0 or hi >= self.num_nodes:
                raise ValueError("indices hold node ids outside [0, num_nodes)")
            if int(self.indptr[-1]) != self.indices.numel() or int(self.indptr[0]) != 0:
                raise ValueError("indptr does not span indices")
        self.node_map = _be.sample_map(self.num_nodes, self.device)
        self._host_pool = []          # pinned read-back buffers for the layer sizes
        self._stream = None

    def batch_seed(self, batch_no):
        """The 64-bit key of batch ``batch_no`` (the sampler's seed and the batch number, mixed)."""
        return (self.seed * 0x9E3779B97F4A7C15 + batch_no * 0xD1B54A32D192ED03 + 1) & 0xFFFFFFFFFFFFFFFF

    def sample(self, seeds, rng_seed=None):
        """Sample the layered sub-graph of ``seeds`` (distinct int64 ids on the device)."""
        return self.sample_async(seeds, rng_seed, stream=torch.cuda.current_stream(self.device)).get()

    def sample_async(self, seeds, rng_seed=None, stream=None):
        """Launch the sampling of one batch on the sampler's side stream (or ``stream``) and return a
        handle; ``handle.get()`` waits for it and returns the batch.  Launching batch i+1 before
        training on batch i keeps the sampling and its size read-back off the training stream.
        Batches of one sampler are sampled one after another (they share the node map)."""
        seeds = torch.as_tensor(seeds, dtype=torch.int64).to(self.device).contiguous()
        if rng_seed is None:
            rng_seed = self.batch_seed(self.batches)
        self.batches += 1
        cur = torch.cuda.current_stream(self.device)
        if stream is None:
            stream = self.stream()
        if stream != cur:
            stream.wait_stream(cur)                                    # seeds may have been produced there
        slot = self._replay_slot(seeds)
        with torch.cuda.stream(stream):
            if slot is not None:
                out = slot.run(self, seeds, rng_seed)
            else:
                out = _be.sample_layers(self.indptr, self.indices, seeds, self.fanout, rng_seed, self.node_map,
                                        emit_view=self.emit_view, view_edges=self.view_edges)
            counts_host = self._host_pool.pop() if self._host_pool else torch.empty(
                2 * len(self.fanout) + 2, dtype=torch.int64, pin_memory=True)
            counts_host.copy_(out[3], non_blocking=True)
            done = torch.cuda.Event()
            done.record(stream)
            y = None if self.labels is None else self.labels[seeds]
        if slot is not None:
            slot.done = done
        return _PendingBatch(self, out, counts_host, done, seeds, y, stream, pooled=slot is not None)

    def stream(self):
        """The sampler's side stream (default priority), made on first use: one that does not share a hardware
        queue with the stream that is current then, or sampling ahead would take turns with the training on it."""
        if self._stream is None:
            self._stream = _be.stream_apart_from([torch.cuda.current_stream(self.device)], self.device)
        return self._stream

    def _replay_slot(self, seeds):
        if not self.replay_slots:
            return None
        slot = self._slots[self._next_slot]
        if slot is None or (slot.graph is None and slot.n_seed != seeds.numel()):
            slot = self._slots[self._next_slot] = _ReplaySlot(seeds.numel(), self.device)
        if slot.n_seed != seeds.numel():
            return None
        self._next_slot = (self._next_slot + 1) % self.replay_slots
        if slot.done is not None:
            slot.done.synchronize()          # the slot's previous batch has been sampled (its seed has been read)
        return slot

    def _finish(self, out, counts_host, seeds, y, stream, pooled=False):
        ptr, idx, s2f = out[:3]
        L = len(self.fanout)
        c = counts_host.tolist()
        self._host_pool.append(counts_host)
        nnl, nel = c[: L + 1], c[L + 1: 2 * L + 1]
        cur = torch.cuda.current_stream(self.device)
        view = None
        if self.emit_view:
            ptrT, rowT, edgeT = out[4], out[5], out[6]
            n_e = max(nel[-1], 1)
            view = _be.BatchView(ptrT[: nnl[L] + 1], rowT[:n_e], None if edgeT is None else edgeT[:n_e],
                                 nnl[L - 1], nnl[L], nel[-1], max_in_degree=c[2 * L + 1])
        if stream != cur:
            # arrays of a replay slot belong to its graph and are never handed back to the allocator
            for t in ((seeds,) if pooled else (ptr, idx, s2f, seeds)) + (() if y is None else (y,)):
                t.record_stream(cur)
            if view is not None and not pooled:
                view.record_stream(cur)
        return SimpleNamespace(
            ptr=ptr[: nnl[L - 1] + 1],
            idx=idx[: nel[-1]],
            sub_to_full=s2f[: nnl[L]],
            num_node_in_layer=torch.tensor(nnl, dtype=torch.int64),   # on the host, as the model reads it
            num_edge_in_layer=list(nel),
            y=y,
            x=None,
            edge_type=None,
            typed_num_node_in_layer=None,
            view=view,
        )


class _PendingBatch:
    """A batch being sampled; ``get()`` returns it once the device has finished."""

    def __init__(self, sampler, out, counts_host, done, seeds, y, stream, pooled=False):
        self._args = (sampler, out, counts_host, done, seeds, y, stream, pooled)
        self._batch = None

    def get(self):
        if self._batch is None:
            sampler, out, counts_host, done, seeds, y, stream, pooled = self._args
            done.synchronize()
            self._batch = sampler._finish(out, counts_host, seeds, y, stream, pooled)
            self._args = None
        return self._batch


class _ReplaySlot:
    """One recorded sampling call: its seeds and its seed key are read from fixed places (a device array, a
    pinned host word), its outputs live in the graph's own memory."""

    def __init__(self, n_seed, device):
        self.n_seed = int(n_seed)
        self.seeds = torch.empty(self.n_seed, dtype=torch.int64, device=device)
        self.key = torch.zeros(1, dtype=torch.int64, pin_memory=True)
        self.graph = None
        self.out = None
        self.done = None

    def run(self, sampler, seeds, rng_seed):
        self.seeds.copy_(seeds)
        k = int(rng_seed) & 0xFFFFFFFFFFFFFFFF
        self.key[0] = k - (1 << 64) if k >= (1 << 63) else k
        if self.graph is None:
            # recorded on a stream of its own (the caller's may be the default stream, which cannot record);
            # the replays run on the caller's
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=torch.cuda.Stream(device=self.seeds.device)):
                self.out = _be.sample_layers(sampler.indptr, sampler.indices, self.seeds, sampler.fanout, 0,
                                             sampler.node_map, emit_view=sampler.emit_view,
                                             view_edges=sampler.view_edges, rng_seed_at=self.key)
            self.graph = graph
        self.graph.replay()
        return self.out
