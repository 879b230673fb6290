"""HistoryTable: per-layer history tables with ring-buffer admission and eviction.

Same public surface as the reference class (/root/reference/hiscache/history_table.py):
``lookup``, ``record_history``, ``evict_by_staleness``, ``evict_by_both``, ``evict_history``,
``show``, and the per-layer attributes (``history_buffer_layered``, ``full_to_history_layered``,
``history_to_full_layered``, ``checkin_iter``, ``cuda_header_layered``, ``sub_to_history``,
``sub_to_history_layered``, ``tmp_history_buffer_layered``, ``history_out``).
Admission runs as one fused gfx950 launch sequence (``hiscache_backend.record_history``); ring slots
are handed out in row order.  The cosine-drift plots of the reference (``self.compare``,
history_table.py:64-70,135-157) are analysis output and are not produced.
"""
from os import path

import torch

import hiscache_backend as _be

from .util import quantile_threshold


class HistoryTable:

    def __init__(self, config, total_num_node=None):
        self.in_channels = config.dl.dataset.feature_dim
        self.out_channels = config.dl.dataset.num_classes
        self.hidden_channels = config.train.model.hidden_dim
        self.num_layers_all = config.train.model.num_layers
        if total_num_node is None:
            total_num_node = int(
                open(path.join(str(config["dl"]["dataset"]["path"]), "processed",
                               "num_nodes.txt")).readline())
        self.total_num_node = int(total_num_node)
        self.device = torch.device(config["dl"]["device"])
        self.store_last_layer = config.history.get("store_last_layer", False)
        self.num_layers = self.num_layers_all - 1 + int(bool(self.store_last_layer))
        self.history_size_layered = self.get_hist_size(config)
        if isinstance(config.history.buffer_size, int):
            self.history_num = [config.history.buffer_size] * self.num_layers
        else:
            assert len(config.history.buffer_size) == self.num_layers
            self.history_num = list(config.history.buffer_size)
        dev = self.device
        self.history_buffer_layered = [
            torch.empty([self.history_num[i], self.history_size_layered[i]], device=dev)
            for i in range(self.num_layers)
        ]
        self.full_to_history_layered = [
            torch.full((self.total_num_node,), -1, dtype=torch.int64, device=dev)
            for _ in range(self.num_layers)
        ]
        self.history_to_full_layered = [
            torch.full((self.history_num[i],), -1, dtype=torch.int64, device=dev)
            for i in range(self.num_layers)
        ]
        self.checkin_iter = [
            torch.full((self.history_num[i],), -1, dtype=torch.int64, device=dev)
            for i in range(self.num_layers)
        ]
        self.cuda_header_layered = [
            torch.zeros([1], dtype=torch.int64, device=dev) for _ in range(self.num_layers)
        ]
        self.method = config.history["method"]
        self.rate = float(config.history["rate"])
        assert self.method in ["random", "grad", "staleness"]
        if self.method != "staleness":
            assert self.rate > 0
        else:
            self.rate = 1
        self.staleness_thres = config.history.staleness_thres
        self.num_used = 0
        self.new_histories = []
        self.history_out = []
        self.graph_struct_norm = int(config.history.graph_struct_norm)
        self.compare = False

    def show(self):
        used_table = []
        for layer_id in range(self.num_layers):
            h2f = self.history_to_full_layered[layer_id]
            used_table.append(int(h2f.shape[0] - h2f.eq(-1).sum()))
        print("used_table", used_table)
        return used_table

    def get_hist_size(self, config):
        """Width of the stored rows per layer (/root/reference/hiscache/history_table.py:79-92)."""
        mtype = config.train.model.type
        if "SAGE" in mtype.upper() or "GCN" == mtype.upper():
            return [self.in_channels] + [self.hidden_channels] * (self.num_layers - 1)
        if "gat" in mtype.lower() or "rgcn" == mtype.lower():
            if not self.store_last_layer:
                return [self.hidden_channels] * self.num_layers
            return [self.hidden_channels] * (self.num_layers - 1) + [self.out_channels]
        raise ValueError("unknown model type " + str(mtype))

    def lookup(self, sub_to_full, num_node_in_layer):
        """Per layer: the slot of every sub-graph node (seeds forced to -1), a compact copy of the
        hit rows and compact ids [-1, 0, -1, 1, ...]
        (/root/reference/hiscache/history_table.py:94-125)."""
        self.tmp_history_buffer_layered = []
        self.sub_to_history_layered = []
        self.sub_to_history = []
        num_seed = int(num_node_in_layer[0])
        for layer_id in range(self.num_layers):
            num_node = int(num_node_in_layer[self.num_layers_all - 1 - layer_id])
            sub_to_history = _be.lookup(self.full_to_history_layered[layer_id],
                                        sub_to_full[:num_node].contiguous())
            sub_to_history[:num_seed] = -1
            mask = sub_to_history != -1
            self.sub_to_history.append(sub_to_history)
            selected = torch.masked_select(sub_to_history, mask)
            tmp_history_buffer = _be.gather_rows(self.history_buffer_layered[layer_id], selected)
            new_id = torch.arange(0, selected.numel(), device=sub_to_history.device)
            compact = torch.full((num_node,), -1, dtype=torch.int64, device=sub_to_history.device)
            compact[mask] = new_id
            if self.method == "grad":
                tmp_history_buffer.requires_grad = True
            self.tmp_history_buffer_layered.append(tmp_history_buffer)
            self.sub_to_history_layered.append(compact)

    def _score(self, grad, batch):
        """L1 row score, optionally scaled by the graph-structure score
        (/root/reference/hiscache/history_table.py:159-172)."""
        if self.method == "grad":
            s = _be.row_scores(grad.contiguous(), _be.NORM_L1)
            if self.graph_struct_norm:
                gs = _be.get_graph_structure_score(batch.ptr, batch.idx, batch.x.shape[0],
                                                   batch.y.shape[0], self.num_layers)
                s = torch.mul(s, gs[:s.shape[0]])
            return s
        if self.method == "random":
            return torch.randn([grad.shape[0]], device=grad.device)
        raise AssertionError("Error record type")

    @torch.no_grad()
    def record_history(self, sub_to_full, batch, glb_iter, used_masks):
        """Admit low-score rows of every layer into its ring
        (/root/reference/hiscache/history_table.py:127-187)."""
        for layer_id in range(self.num_layers):
            if self.history_buffer_layered[layer_id].shape[0] == 0:
                continue
            num_node = int(batch.num_node_in_layer[self.num_layers_all - 1 - layer_id])
            his = self.history_out[layer_id][:num_node]
            grad = (self.history_out[layer_id].grad)[:num_node]
            record_sum = self._score(grad, batch)
            thres = quantile_threshold(record_sum, self.rate)
            _be.record_history(his.detach().contiguous(), self.history_buffer_layered[layer_id],
                               used_masks[layer_id + 1], sub_to_full, self.sub_to_history[layer_id],
                               self.history_to_full_layered[layer_id],
                               self.full_to_history_layered[layer_id],
                               self.cuda_header_layered[layer_id], record_sum, thres,
                               self.checkin_iter[layer_id], glb_iter)

    def evict_by_staleness(self, glb_iter, staleness_thres):
        """Un-map slots with -1 < checkin <= glb_iter - limit
        (/root/reference/hiscache/history_table.py:189-200)."""
        if isinstance(staleness_thres, int):
            staleness_thres = [staleness_thres] * self.num_layers
        for layer_id in range(self.num_layers):
            _be.evict(self.checkin_iter[layer_id], self.history_to_full_layered[layer_id],
                      self.full_to_history_layered[layer_id], glb_iter - staleness_thres[layer_id])

    def evict_by_both(self, batch, glb_iter, staleness_thres):
        """Evict cached rows whose score is in the top ``rate`` quantile, then by staleness
        (/root/reference/hiscache/history_table.py:202-251); one launch per table."""
        if self.method == "staleness":
            self.evict_by_staleness(glb_iter, staleness_thres)
            return
        if isinstance(staleness_thres, int):
            staleness_thres = [staleness_thres] * self.num_layers
        for layer_id in range(self.num_layers):
            if self.history_buffer_layered[layer_id].shape[0] == 0:
                continue
            num_node = int(batch.num_node_in_layer[self.num_layers_all - 1 - layer_id])
            grad = (self.history_out[layer_id].grad)[:num_node]
            evict_sum = self._score(grad, batch)
            thres = quantile_threshold(evict_sum, 1 - self.rate)
            _be.evict(self.checkin_iter[layer_id], self.history_to_full_layered[layer_id],
                      self.full_to_history_layered[layer_id], glb_iter - staleness_thres[layer_id],
                      sub2slot=self.sub_to_history[layer_id][:num_node].contiguous(), score=evict_sum, thres=thres)

    def evict_history(self, batch, glb_iter):
        self.evict_by_both(batch, glb_iter, self.staleness_thres)
