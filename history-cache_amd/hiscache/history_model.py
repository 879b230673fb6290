"""GraphSAGE with a history-aware aggregation layer.

Same classes and forward wiring as the reference's SAGE path
(/root/reference/hiscache/history_model.py:54-184): ``MySageConvHistory``, ``HistorySAGE`` and
``get_model``.  Aggregation (with and without history) runs through ``hiscache_backend``; the
dense layers are stock PyTorch.  The plain mean that the reference takes from
``cxgnncomp.sage_mean_forward`` (history_model.py:90) is the same kernel with no history map.
The RGCN / DGL wrappers depend on external operator libraries and are not part of this module.
"""
import torch
import torch.nn.functional as F

import hiscache_backend


class MySageConvHistory(torch.nn.Module):

    def __init__(self, in_channels, hidden_channels, need_grad, root_weight: bool = True,
                 bias: bool = True):
        super().__init__()
        self.in_channels = in_channels
        self.hidden_channels = hidden_channels
        self.root_weight = root_weight
        self.lin_l = torch.nn.Linear(in_channels, hidden_channels, bias=bias)
        if self.root_weight:
            self.lin_r = torch.nn.Linear(in_channels, hidden_channels, bias=False)
        self.reset_parameters()
        self.need_grad = need_grad

    def reset_parameters(self):
        self.lin_l.reset_parameters()
        if self.root_weight:
            self.lin_r.reset_parameters()

    def forward(self, x, ptr, idx, history_map, history_buffer, history_size, num_node):
        num_node = int(num_node)
        # history_size == 0 selects the plain mean inside the operator
        out = hiscache_backend.aggr_forward_history(x, ptr, idx, history_map, history_buffer,
                                                    history_size, num_node)
        his = out
        if self.need_grad and self.training and history_size > 0:
            his.retain_grad()
        out = self.lin_l(out)
        if self.root_weight:
            if num_node != 0:
                out = out + self.lin_r(x[:num_node])
            else:
                out = out + self.lin_r(x)
        return out, his


class HistorySAGE(torch.nn.Module):

    def __init__(self, in_channels, hidden_channels, out_channels, num_layers, dropout, graph_type,
                 config, table, **kwargs):
        super().__init__()
        self.in_channels = in_channels
        self.hidden_channels = hidden_channels
        self.out_channels = out_channels
        self.graph_type = graph_type
        self.bns = torch.nn.ModuleList()
        self.num_layers = num_layers
        for _ in range(self.num_layers - 1):
            self.bns.append(torch.nn.BatchNorm1d(hidden_channels))
        self.dropout = dropout
        self.table = table
        self.init_convs(**kwargs)

    def forward(self, batch):
        x = batch.x
        none = torch.empty(0, device=x.device)
        for i, conv in enumerate(self.convs[:-1]):
            n = batch.num_node_in_layer[self.num_layers - 1 - i]
            if self.training and i == self.num_layers - 2:
                # the layer whose output is one hop from the seeds uses (and produces) history
                x, his = conv(x, batch.ptr, batch.idx, self.table.sub2embed,
                              self.table.cached_embedding, self.hidden_channels, n)
                self.table.produced_embedding = his
            else:
                x, his = conv(x, batch.ptr, batch.idx, none, none, 0, n)
            x = self.bns[i](x)
            x = F.relu(x)
            x = F.dropout(x, p=self.dropout, training=self.training)
        x, his = self.convs[-1](x, batch.ptr, batch.idx, none, none, 0, batch.num_node_in_layer[0])
        return x.log_softmax(dim=-1)

    def init_convs(self, **kwargs):
        need_grad = self.table.method == "grad"
        self.convs = torch.nn.ModuleList()
        self.convs.append(
            self.init_history_conv(self.in_channels, self.hidden_channels, need_grad=need_grad, **kwargs))
        for _ in range(self.num_layers - 2):
            self.convs.append(
                self.init_history_conv(self.hidden_channels, self.hidden_channels, need_grad=need_grad,
                                       **kwargs))
        if self.num_layers > 1:
            self.last_layer_history = False
            self.convs.append(
                self.init_history_conv(self.hidden_channels, self.out_channels, need_grad=need_grad,
                                       **kwargs))

    def init_history_conv(self, in_channels, out_channels, **kwargs):
        assert "need_grad" in kwargs
        return MySageConvHistory(in_channels, out_channels, **kwargs)

    def reset_parameters(self):
        for conv in self.convs:
            conv.reset_parameters()
        for bn in self.bns:
            bn.reset_parameters()


model_dict = {"sage": HistorySAGE}
graph_type_dict = {"cxg": "CSR_Layer", "dgl": "DGL"}


def get_model(config, table):
    """Model factory with the reference's signature (/root/reference/hiscache/history_model.py:446-470)."""
    mtype = config.train.model.type.lower()
    if mtype not in model_dict:
        raise NotImplementedError(f"model type {mtype!r}: only the SAGE path is provided")
    return model_dict[mtype](config.dl.dataset.feature_dim, config.train.model.hidden_dim,
                             config.dl.dataset.num_classes, config.train.model.num_layers,
                             config.train.model.dropout, graph_type_dict[config.train.type.lower()],
                             config, table)
