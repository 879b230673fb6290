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

    def __init__(self, indptr, indices, fanout, labels=None, seed=0, device="cuda:0", validate=True):
        """``indptr`` / ``indices``: CSR of the full graph (int64; moved to ``device``).  ``fanout[k]``
        neighbours are drawn, without replacement, for nodes first reached at hop k."""
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
        self._counts_host = torch.empty(2 * len(self.fanout) + 1, dtype=torch.int64, pin_memory=True)

    def batch_seed(self, batch_no):
        """The 64-bit key of batch ``batch_no`` (the sampler's seed and the batch number, mixed)."""
        return (self.seed * 0x9E3779B97F4A7C15 + batch_no * 0xD1B54A32D192ED03 + 1) & 0xFFFFFFFFFFFFFFFF

    def sample(self, seeds, rng_seed=None):
        """Sample the layered sub-graph of ``seeds`` (distinct int64 ids on the device)."""
        seeds = torch.as_tensor(seeds, dtype=torch.int64).to(self.device).contiguous()
        if rng_seed is None:
            rng_seed = self.batch_seed(self.batches)
        self.batches += 1
        L = len(self.fanout)
        ptr, idx, s2f, counts = _be.sample_layers(self.indptr, self.indices, seeds, self.fanout, rng_seed,
                                                  self.node_map)
        self._counts_host.copy_(counts, non_blocking=True)
        torch.cuda.current_stream(self.device).synchronize()
        c = self._counts_host.tolist()
        nnl, nel = c[: L + 1], c[L + 1:]
        return SimpleNamespace(
            ptr=ptr[: nnl[L - 1] + 1],
            idx=idx[: nel[-1]],
            sub_to_full=s2f[: nnl[L]],
            num_node_in_layer=torch.tensor(nnl, dtype=torch.int64),   # on the host, as the model reads it
            num_edge_in_layer=list(nel),
            y=None if self.labels is None else self.labels[seeds],
            x=None,
            edge_type=None,
            typed_num_node_in_layer=None,
        )
