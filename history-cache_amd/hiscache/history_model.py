"""GraphSAGE and RGCN with a history-aware aggregation layer.

Same classes and forward wiring as the reference (/root/reference/hiscache/history_model.py):
``MySageConvHistory`` / ``HistorySAGE`` (:54-184), ``MyRGCNConvHistory2`` / ``HistoryRGCN``
(:220-431) and ``get_model`` (:446-470).  Aggregation (with and without history) runs through
``hiscache_backend``; the dense layers are stock PyTorch.  The plain mean that the reference takes
from ``cxgnncomp.sage_mean_forward`` (history_model.py:90) is the same kernel with no history map.
The relational layer replaces ``cxgnncomp.RGCNOP_sorted`` (:266) by a typed gather-reduce -- the
mean kernel over (row, relation) virtual rows -- followed by one GEMM; the result is the same
quantity, sum_j x[src_j] @ W[rel_j] / deg.  The DGL wrapper is not part of this module.
"""
import weakref

import torch
import torch.nn.functional as F

import hiscache_backend


class _GradSink:
    """Where the fused convolution leaves the gradient that reached its aggregation output: the
    tensor the model hands to the cache as ``produced_embedding`` (held weakly)."""
    __slots__ = ("target",)

    def __init__(self):
        self.target = None


# rocBLAS's kernel choice for a weight gradient g^T x ([H, n] x [n, F], n = rows of a sampled layer) is
# erratic in n: measured on MI355X with H = 256, the single GEMM takes 52 us at n = 25 800 and F = 128,
# 353 us at F = 256, 1.5 ms at n = 55 000 and 2.4 ms at n = 89 000 (one or two tiles walking the whole
# inner dimension).  As a batched GEMM over slabs of 1 024 rows plus a sum over the slabs it takes 42, 69,
# 72 - 131 and 107 - 193 us: linear in n.  Below this many rows the single GEMM is used (21 us at 5 800).
_WGRAD_SLAB_ROWS = 1024
_WGRAD_SPLIT_MIN_ROWS = 8192
# The library's own kernel (hc_weight_grad: both operands of a SAGE layer in one pair of launches, 59 us at
# n = 25 800 and F = 128, 102 us at n = 55 000) takes over from this many rows when the widths fit it.
_WGRAD_KERNEL_MIN_ROWS = 2048


def _weight_grad(g, x):
    """g^T @ x for g [n, H], x [n, F] (both contiguous): the gradient of a linear layer's weight."""
    n = g.shape[0]
    if n < _WGRAD_SPLIT_MIN_ROWS:
        return g.t() @ x
    S = n // _WGRAD_SLAB_ROWS
    m = n // S * S
    out = torch.bmm(g[:m].view(S, m // S, -1).transpose(1, 2), x[:m].view(S, m // S, -1)).sum(0)
    if m < n:
        out.addmm_(g[m:].t(), x[m:])
    return out


_ones_cache = {}


def _column_sums(g):
    """g.sum(0) as a matrix-vector product with a cached vector of ones: torch's column reduction of a tall
    [n, H] matrix takes 25 us at n = 1 000 (one block per few columns walks all rows), the GEMV 12 us."""
    n = g.shape[0]
    key = (g.device, g.dtype)
    ones = _ones_cache.get(key)
    if ones is None or ones.numel() < n:
        size = 1024
        while size < n:
            size <<= 1
        ones = _ones_cache[key] = torch.ones(size, dtype=g.dtype, device=g.device)
    return torch.mv(g.t(), ones[:n])


class _SageConvFunction(torch.autograd.Function):
    """``lin_l(aggregate(x)) + lin_r(x[:n])`` as ONE autograd node.

    Spelled with separate operators (as /root/reference/hiscache/history_model.py:85-100 does) the
    backward of a layer runs, besides its GEMMs, a zero fill and a copy for the gradient of the slice
    ``x[:n]`` and an add that joins it with the aggregation's input gradient.  Here the aggregation's
    input gradient is written first and the root term's gradient is accumulated into its first n rows
    by the GEMM itself.  The aggregation output is returned as a second, non-differentiable result;
    the gradient that reaches it (what ``retain_grad()`` keeps in the unfused spelling) is stored in
    its ``.grad`` during backward when a sink is given."""

    @staticmethod
    def forward(ctx, x, w_l, b_l, w_r, ptr, idx, hmap, hbuf, hsize, num_node, num_edge, sink, view=None):
        be = hiscache_backend
        R = int(num_node) if num_node else ptr.numel() - 1
        agg = be._aggr_fwd(be.SUBST_ROW, ptr, idx, x, hmap, hbuf, hsize, None, R)
        # plain GEMMs and a separate bias add: a GEMM with a bias epilogue goes to hipBLASLt whatever
        # library is preferred, and its per-shape set-up costs the host more than the extra launch
        out = agg @ w_l.t()
        if w_r is not None:
            root = x[:R] if x.dtype == agg.dtype else x[:R].to(agg.dtype)
            out.addmm_(root, w_r.t())
        if b_l is not None:
            out += b_l
        ctx.save_for_backward(x, agg, w_l, w_r if w_r is not None else w_l.new_empty(0))
        ctx.hc = (ptr, idx, hmap, hsize, R, num_edge, b_l is not None, w_r is not None, sink)
        ctx.view = view if view is not None and view.covers(R, x.shape[0]) else None
        ctx.mark_non_differentiable(agg)
        # no zero tensor for the gradient of `agg`, which never has one (a fill of [R, F] per layer otherwise)
        ctx.set_materialize_grads(False)
        return out, agg

    @staticmethod
    def backward(ctx, g_out, _g_agg_unused):
        be = hiscache_backend
        ptr, idx, hmap, hsize, R, num_edge, has_bias, has_root, sink = ctx.hc
        x, agg, w_l, w_r = ctx.saved_tensors
        if g_out is None:                                     # the layer's output did not reach the loss
            return (None,) * 13
        g_out = g_out.contiguous()
        need = ctx.needs_input_grad
        g_agg = g_out @ w_l                                   # gradient reaching the aggregation output
        if sink is not None and sink.target is not None:
            his = sink.target()
            if his is not None:
                his.grad = g_agg
        g_bl = _column_sums(g_out) if has_bias and need[2] else None
        g_wl = g_wr = None
        root = None
        if has_root and need[3]:
            root = x[:R] if x.dtype == g_out.dtype else x[:R].to(g_out.dtype)
        if need[1] and root is not None and R >= _WGRAD_KERNEL_MIN_ROWS and be.weight_grad_supported(g_out, agg):
            g_wl, g_wr = be.weight_grad(g_out, agg, root)          # both products in one pair of launches
        else:
            if need[1]:
                g_wl = _weight_grad(g_out, agg)
            if root is not None:
                g_wr = _weight_grad(g_out, root)
        g_x = None
        if need[0]:
            n_src = x.shape[0]
            if ctx.view is not None:          # the batch came with its transposed view: none is built here
                g_x, _ = be._aggr_bwd_batch_view(ptr, ctx.view, g_agg, hmap, None, hsize, R, n_src,
                                                 want_hist_grad=False)
            else:
                tr = be.build_transpose(ptr, idx, hmap, R, n_src, num_edge=num_edge, want_edges=False)
                g_x, _, _ = be._aggr_bwd(ptr, idx, tr, g_agg, hmap, None, x, False, None, hsize, R, n_src,
                                         want_hist_grad=False)
            if has_root:
                g_x[:R].addmm_(g_out, w_r)
            if g_x.dtype != x.dtype:
                g_x = g_x.to(x.dtype)
        return g_x, g_wl, g_bl, g_wr, None, None, None, None, None, None, None, None, None


def bn_relu(x, bn, bias=None, fused=True, n_dev=None):
    """``F.relu(bn(x + bias))`` (/root/reference/hiscache/history_model.py:139-140).  In training mode on
    the GPU this is one autograd node over the library's epilogue kernels (two launches forward, two
    backward, against eight and four operator by operator); ``bias`` then must NOT have been added to
    ``x`` yet.  Otherwise the torch operators run.  ``bn``'s running statistics and batch counter are
    updated as ``torch.nn.BatchNorm1d.forward`` updates them.  ``n_dev`` (one int64 on the device; recorded
    iterations over padded batches): the number of rows of ``x`` that are in use."""
    be = hiscache_backend
    if not (fused and bn.training and x.dim() == 2 and be.bn_relu_supported(x, x.shape[1])
            and x.shape[0] > 1):
        if n_dev is not None:
            raise ValueError("a row count on the device needs the fused epilogue (training mode, fp32 on the GPU)")
        if bias is not None:
            x = x + bias
        return F.relu(bn(x))
    momentum = 0.0 if bn.momentum is None else bn.momentum
    track = bn.track_running_stats and bn.running_mean is not None
    counter = None
    if track and bn.num_batches_tracked is not None:
        if bn.momentum is None:                       # cumulative moving average: the count is needed here
            bn.num_batches_tracked.add_(1)
            momentum = 1.0 / float(bn.num_batches_tracked)
        else:
            counter = bn.num_batches_tracked          # incremented by the statistics kernel
    return be.bias_bn_relu(x, bias, bn.weight, bn.bias, bn.running_mean if track else None,
                           bn.running_var if track else None, momentum, bn.eps, counter, n_dev)


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

    # one autograd node per layer (see _SageConvFunction); False spells the layer operator by operator
    fused = True

    def forward(self, x, ptr, idx, history_map, history_buffer, history_size, num_node, num_edge=None,
                add_bias=True, view=None):
        """``add_bias=False`` leaves ``lin_l``'s bias to the caller, who hands it to the normalisation
        that follows (see ``bn_relu``).  ``view``: the batch's shared transposed view
        (``hiscache_backend.BatchView``), when the loader emitted one."""
        num_node = int(num_node)
        # (no rows to substitute from: the no-cache mode hands over a map of -1 and an empty buffer)
        use_hist = (history_size > 0 and history_map is not None and history_map.numel() > 0
                    and history_buffer is not None and history_buffer.numel() > 0)
        if self.fused and x.is_cuda and not (use_hist and history_buffer.requires_grad):
            sink = None
            if self.need_grad and self.training and history_size > 0:
                sink = _GradSink()
            out, his = _SageConvFunction.apply(
                x, self.lin_l.weight, self.lin_l.bias if add_bias else None,
                self.lin_r.weight if self.root_weight else None, ptr, idx,
                history_map if use_hist else None, history_buffer if use_hist else None,
                int(history_size) if use_hist else 0, num_node, num_edge, sink, view)
            if sink is not None:
                sink.target = weakref.ref(his)
            return out, his
        # history_size == 0 selects the plain mean inside the operator; num_edge (optional, beyond the
        # reference) bounds the edge slots of these rows inside the mini-batch's shared CSR
        out = hiscache_backend.aggr_forward_history(x, ptr, idx, history_map, history_buffer,
                                                    history_size, num_node, num_edge, view)
        his = out
        if self.need_grad and self.training and history_size > 0:
            his.retain_grad()
        out = self.lin_l(out) if add_bias else F.linear(out, self.lin_l.weight)
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

    # bias + batch norm + ReLU of a hidden layer as one autograd node (see bn_relu); False spells them
    # with torch operators
    fused_epilogue = True

    def forward(self, batch):
        x = batch.x
        none = torch.empty(0, device=x.device)
        nel = getattr(batch, "num_edge_in_layer", None)      # edges of the first num_node_in_layer[k] rows
        view = getattr(batch, "view", None)                  # shared transposed view, if the loader emitted it
        # a batch padded to fixed sizes for a recorded iteration carries its real sizes on the device
        dev = getattr(batch, "dev", None)
        # ... and row offsets per layer, flat behind the layer's real rows (see hiscache.RecordedIteration)
        ptrs = getattr(batch, "ptr_of_layer", None)
        for i, conv in enumerate(self.convs[:-1]):
            k = self.num_layers - 1 - i
            n = batch.num_node_in_layer[k]
            ne = None if nel is None else int(nel[k])
            ptr = batch.ptr if ptrs is None else ptrs[k]
            # the bias of lin_l goes to the normalisation's kernels instead of a launch of its own
            defer = self.fused_epilogue and conv.fused and self.training and x.is_cuda
            if self.training and i == self.num_layers - 2:
                # the layer whose output is one hop from the seeds uses (and produces) history
                x, his = conv(x, ptr, batch.idx, self.table.sub2embed,
                              self.table.cached_embedding, self.hidden_channels, n, ne, add_bias=not defer,
                              view=view)
                self.table.produced_embedding = his
            else:
                x, his = conv(x, ptr, batch.idx, none, none, 0, n, ne, add_bias=not defer, view=view)
            x = bn_relu(x, self.bns[i], conv.lin_l.bias if defer else None, fused=self.fused_epilogue,
                        n_dev=None if dev is None else dev.nnl[k])
            x = F.dropout(x, p=self.dropout, training=self.training)
        x, his = self.convs[-1](x, batch.ptr if ptrs is None else ptrs[0], batch.idx, none, none, 0,
                                batch.num_node_in_layer[0], None if nel is None else int(nel[0]), view=view)
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


def typed_csr(ptr, idx, edge_types, num_rel, num_node, used_mask=None, n_src=None):
    """Group the edges of the first ``num_node`` rows by (row, relation): returns (ptr2, idx2, cnt, deg)
    where virtual row r*num_rel+k of (ptr2, idx2) holds row r's edges of relation k in their original
    order, cnt[num_node, num_rel] are the group sizes and deg[num_node] the full row degrees.
    ``edge_types`` covers at least the edges of those rows (it may be longer).  Edges whose source is
    not in ``used_mask`` are dropped, as the reference drops them by giving them an extra relation
    (/root/reference/hiscache/history_model.py:248-250).  One library call: nothing is sorted and no
    device value is read back."""
    if n_src is None:
        n_src = int(used_mask.shape[0]) if used_mask is not None else (1 << 62)
    return hiscache_backend.typed_csr(ptr, idx, edge_types.to(torch.int64).contiguous(), num_rel, num_node,
                                      n_src, used_mask)


def edge_types_by_node_ranges(ptr, idx, sub_to_full, num_node, type_bounds, pair_to_rel):
    """Relation of every edge of the first ``num_node`` rows from the node types of its ends; a node's
    type is the range of ``type_bounds`` its full id falls into (mag240M stores papers, authors and
    institutions in consecutive id ranges).  ``pair_to_rel[type(dst), type(src)]`` gives the relation.
    Stands in for ``cxgnncomp_backend.gen_edge_type_mag240m``
    (/root/reference/hiscache/history_model.py:356), whose exact numbering is not available here.
    ``type_bounds`` and ``pair_to_rel`` may be device tensors (no copy) or host sequences."""
    dev = ptr.device
    bounds = type_bounds if isinstance(type_bounds, torch.Tensor) else torch.as_tensor(
        type_bounds, dtype=torch.int64, device=dev)
    table = pair_to_rel if isinstance(pair_to_rel, torch.Tensor) else torch.as_tensor(
        pair_to_rel, dtype=torch.int64, device=dev)
    return hiscache_backend.edge_types_by_ranges(ptr, idx, sub_to_full, num_node, bounds.contiguous(),
                                                 table.contiguous())


# Shapes of the relational layer's GEMMs, [n, K*F] x [K*F, H] with n in the thousands, for which
# rocBLAS's single-GEMM kernels run at a third of what its batched kernels reach (measured on MI355X,
# n = 4 200, K*F = 3 840, H = 256, fp32): forward 214 us as one GEMM, 85 us as K GEMMs over the
# relations plus a sum; weight gradient 230 us as one GEMM, 111 us as 8 GEMMs over slabs of rows plus a
# sum.  Below this inner size one GEMM is the faster spelling.
_REL_SPLIT_MIN_INNER = 2048
_REL_WGRAD_SLABS = 8


def _rel_matmul(agg, weight):
    """sum_k agg[:, k, :] @ weight[k]; agg is [n, K, F] (contiguous), weight [K, F, H]."""
    n, K, Fin = agg.shape
    if K * Fin >= _REL_SPLIT_MIN_INNER and K > 1:
        return torch.bmm(agg.transpose(0, 1), weight).sum(0)
    return agg.reshape(n, K * Fin) @ weight.reshape(K * Fin, -1)


def _rel_weight_grad(agg, g):
    """agg^T @ g in the weight's layout: agg [n, K, F], g [n, H] -> [K, F, H]."""
    n, K, Fin = agg.shape
    a2 = agg.reshape(n, K * Fin)
    S = max(_REL_WGRAD_SLABS, n // _WGRAD_SLAB_ROWS)
    m = n // S * S
    if K * Fin < _REL_SPLIT_MIN_INNER or m == 0:
        return (a2.t() @ g).view(K, Fin, -1)
    out = torch.bmm(a2[:m].view(S, m // S, K * Fin).transpose(1, 2), g[:m].view(S, m // S, -1)).sum(0)
    if m < n:
        out.addmm_(a2[m:].t(), g[m:])
    return out.view(K, Fin, -1)


class _RgcnConvFunction(torch.autograd.Function):
    """The relational convolution as ONE autograd node: (row, relation) grouping, aggregation with the
    groups' shares of the row mean as edge weights (no pass that rescales group means), the GEMM with
    the relation weights and the history substitution.  Backward computes the weight gradient and,
    only when the layer's input needs one (never at the feature layer), the input gradient through
    the weighted aggregation's transposed view."""

    @staticmethod
    def forward(ctx, x, weight, ptr, idx, edge_types, used_mask, hmap, hbuf, num_node, view=None, sink=None):
        be = hiscache_backend
        ctx.sink = sink
        R = int(num_node)
        K, Fin, H = weight.shape
        ptr2, idx2, _cnt, _deg, w2 = be.typed_csr(ptr, idx, edge_types, K, R, x.shape[0], used_mask,
                                                  want_weights=True)
        agg = be._aggr_fwd(be.SUBST_ROW, ptr2, idx2, x, None, None, 0, w2, R * K).view(R, K, Fin)
        out = _rel_matmul(agg, weight)
        hit = None
        if hmap is not None:
            hit = (hmap[:R] != -1).unsqueeze(1)
            out = torch.where(hit, hbuf[:R].to(out.dtype), out)
        ctx.save_for_backward(x, agg, weight, ptr2, idx2, w2, hit if hit is not None else x.new_empty(0))
        ctx.hc = (R, hit is not None, min(int(edge_types.numel()), int(idx.numel())))
        # the batch's shared transposed view (with edge slots) serves backward directly
        ctx.shared = (ptr, edge_types, used_mask, view) if be.typed_batch_view_supported(
            view, R, x.shape[0], Fin) else None
        return out

    @staticmethod
    def backward(ctx, g):
        be = hiscache_backend
        x, agg, weight, ptr2, idx2, w2, hit = ctx.saved_tensors
        R, has_hit, E = ctx.hc
        K, Fin, H = weight.shape
        g = g.contiguous()
        if ctx.sink is not None and ctx.sink.target is not None:
            his = ctx.sink.target()
            if his is not None:
                his.grad = g                          # what retain_grad() would keep, without its copy
        if has_hit:                                   # rows taken from the history pass nothing back
            g = g.masked_fill(hit, 0.0)
        g_w = _rel_weight_grad(agg, g) if ctx.needs_input_grad[1] else None
        g_x = None
        if ctx.needs_input_grad[0]:
            g_agg = (g @ weight.reshape(K * Fin, H).t()).view(R * K, Fin)
            n_src = x.shape[0]
            if ctx.shared is not None:
                ptr, edge_types, used_mask, view = ctx.shared
                g_x = be._aggr_bwd_typed_batch_view(ptr, view, edge_types, K, used_mask, g_agg, R, n_src)
            else:
                tr = be.build_transpose(ptr2, idx2, None, R * K, n_src, num_edge=E, want_edges=True)
                g_x, _, _ = be._aggr_bwd(ptr2, idx2, tr, g_agg, None, w2, x, False, None, 0, R * K, n_src,
                                         want_hist_grad=False)
            if g_x.dtype != x.dtype:
                g_x = g_x.to(x.dtype)
        return g_x, g_w, None, None, None, None, None, None, None, None, None


class MyRGCNConvHistory2(torch.nn.Module):
    """Relational convolution with history substitution: out[r] = sum_j x[src_j] @ W[rel_j] / deg(r),
    rows with a cached embedding take it instead
    (/root/reference/hiscache/history_model.py:220-278)."""

    def __init__(self, in_channels, hidden_channels, num_rel, need_grad):
        super().__init__()
        self.in_channels = in_channels
        self.hidden_channels = hidden_channels
        self.num_rel = num_rel
        self.linear = torch.nn.Parameter(torch.empty(num_rel, in_channels, hidden_channels))
        # the reference registers the same tensor a second time under this name
        # (/root/reference/hiscache/history_model.py:233-236), so its checkpoints hold both keys
        self.register_parameter("rel_weight", self.linear)
        self.reset_parameters()
        self.need_grad = need_grad
        self._count_of = None

    def reset_parameters(self):
        # glorot, as torch_geometric.nn.inits.glorot does for a [K, in, out] weight
        bound = (6.0 / (self.linear.size(-2) + self.linear.size(-1))) ** 0.5
        torch.nn.init.uniform_(self.linear, -bound, bound)

    # one autograd node per layer (see _RgcnConvFunction); False spells the layer operator by operator
    fused = True

    @property
    def last_count(self):
        """Per-relation edge counts of the last call, as the reference takes them in front of its
        sorted operator (/root/reference/hiscache/history_model.py:260); computed when asked for."""
        if self._count_of is None:
            return None
        return hiscache_backend.count_num(self._count_of, self.num_rel)

    def forward(self, x, ptr, idx, edge_types, count, history_map, history_buffer, used_mask, history_size,
                num_node, view=None):
        num_node = int(num_node)
        K = self.num_rel
        edge_types = edge_types.to(torch.int64).contiguous()
        self._count_of = edge_types
        # (no rows to substitute from: the no-cache mode hands over a map of -1 and an empty buffer)
        use_hist = (history_size > 0 and history_map is not None and history_map.numel() > 0
                    and history_buffer is not None and history_buffer.numel() > 0)
        if self.fused and x.is_cuda and not (use_hist and history_buffer.requires_grad):
            # the gradient that reaches the layer's output is handed to ``his.grad`` by the node's backward
            sink = _GradSink() if (self.need_grad and self.training and history_size > 0) else None
            out = _RgcnConvFunction.apply(x, self.linear, ptr, idx, edge_types, used_mask,
                                          history_map if use_hist else None,
                                          history_buffer if use_hist else None, num_node, view, sink)
            his = out
            if sink is not None:
                sink.target = weakref.ref(his)
                his._hc_grad_sink = True
            return out, his
        ptr2, idx2, cnt, deg = typed_csr(ptr, idx, edge_types, K, num_node, used_mask, n_src=x.shape[0])
        none = torch.empty(0, device=x.device)
        # mean over every (row, relation) group; cnt/deg turns the group means into the row's share
        agg = hiscache_backend.aggr_forward_history(x, ptr2, idx2, none, none, 0, num_node * K)
        scale = cnt.to(torch.float32) / deg.clamp(min=1).to(torch.float32)[:, None]
        agg = agg.view(num_node, K, -1) * scale[:, :, None]
        out = agg.reshape(num_node, -1) @ self.linear.reshape(K * self.in_channels, self.hidden_channels)
        if history_size > 0:
            hit = (history_map[:num_node] != -1)[:, None]
            out = torch.where(hit, history_buffer[:num_node].to(out.dtype), out)
        his = out
        if self.need_grad and self.training and history_size > 0:
            his.retain_grad()
        return out, his


MyRGCNConvHistory = MyRGCNConvHistory2


class HistoryRGCN(torch.nn.Module):
    """Forward wiring of /root/reference/hiscache/history_model.py:329-431."""

    def __init__(self, in_channels, hidden_channels, out_channels, num_layers, dropout, graph_type, config,
                 table, **kwargs):
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
        self.num_rel = kwargs["num_rel"]
        self.dataset_name = kwargs.get("dataset_name", "")
        self.gen_rel = self.dataset_name == "rmag240m"
        if self.gen_rel:
            self.num_rel = 5
        # node-type id ranges and the (dst type, src type) -> relation table used when gen_rel
        self.type_bounds = kwargs.get("type_bounds")
        self.pair_to_rel = kwargs.get("pair_to_rel")
        need_grad = self.table.method == "grad"
        self.convs = torch.nn.ModuleList()
        self.convs.append(MyRGCNConvHistory2(in_channels, hidden_channels, self.num_rel, need_grad))
        for _ in range(self.num_layers - 2):
            self.convs.append(MyRGCNConvHistory2(hidden_channels, hidden_channels, self.num_rel, need_grad))
        if self.num_layers > 1:
            self.last_layer_history = False
            self.convs.append(MyRGCNConvHistory2(hidden_channels, out_channels, self.num_rel, need_grad))

    fused_epilogue = True

    def edge_types(self, batch):
        L = self.num_layers
        if getattr(batch, "edge_type", None) is not None:
            return batch.edge_type
        if self.gen_rel and self.type_bounds is not None:
            if not isinstance(self.type_bounds, torch.Tensor):     # moved to the device once
                dev = batch.ptr.device
                self.type_bounds = torch.as_tensor(self.type_bounds, dtype=torch.int64, device=dev)
                self.pair_to_rel = torch.as_tensor(self.pair_to_rel, dtype=torch.int64, device=dev)
            return edge_types_by_node_ranges(batch.ptr, batch.idx, batch.sub_to_full,
                                             int(batch.num_node_in_layer[L - 1]), self.type_bounds,
                                             self.pair_to_rel)
        return torch.randint(0, self.num_rel, (batch.num_edge_in_layer[L - 1],), device=batch.ptr.device)

    def forward(self, batch):
        x = batch.x
        L = self.num_layers
        etypes = self.edge_types(batch)
        none = torch.empty(0, device=x.device)
        # the used masks belong to the training lookup of this batch; an evaluation lookup
        # (``feature_cache_only``) prunes nothing and computes none (the reference keeps reading the last
        # training batch's masks there, /root/reference/hiscache/history_model.py:373-396)
        masks = self.table.used_masks if self.training else None
        view = getattr(batch, "view", None)                  # shared transposed view, if the loader emitted it
        dev = getattr(batch, "dev", None)                    # a padded batch carries its real sizes on the device
        ptrs = getattr(batch, "ptr_of_layer", None)          # ... and row offsets per layer (see HistorySAGE.forward)
        for i, conv in enumerate(self.convs[:-1]):
            n = batch.num_node_in_layer[L - 1 - i]
            et = etypes[: batch.num_edge_in_layer[L - 1 - i]]
            um = masks[i] if masks is not None else None
            ptr = batch.ptr if ptrs is None else ptrs[L - 1 - i]
            if self.training and i == L - 2:
                x, his = conv(x, ptr, batch.idx, et, None, self.table.sub2embed,
                              self.table.cached_embedding, um, self.hidden_channels, n, view=view)
                self.table.produced_embedding = his
                if not getattr(his, "_hc_grad_sink", False):
                    self.table.produced_embedding.retain_grad()
            else:
                x, his = conv(x, ptr, batch.idx, et, None, none, none, um, 0, n, view=view)
            x = bn_relu(x, self.bns[i], None, fused=self.fused_epilogue,
                        n_dev=None if dev is None else dev.nnl[L - 1 - i])
            x = F.dropout(x, p=self.dropout, training=self.training)
        um = masks[-2] if masks is not None else None
        x, his = self.convs[-1](x, batch.ptr if ptrs is None else ptrs[0], batch.idx,
                                etypes[: batch.num_edge_in_layer[0]], None, none, none, um, 0,
                                batch.num_node_in_layer[0], view=view)
        return x.log_softmax(dim=-1)

    def reset_parameters(self):
        for conv in self.convs:
            conv.reset_parameters()
        for bn in self.bns:
            bn.reset_parameters()


def prefer_low_latency_gemm(enable=True):
    """Route torch's GEMMs to rocBLAS (``enable``) or back to torch's default choice.

    Sampled batches give every GEMM of an iteration a row count that was never seen before.
    hipBLASLt, torch's default on this GPU, selects a kernel per problem shape, which costs the host
    about 80 us per call for a new shape (20 us for a repeated one); rocBLAS costs 11 - 17 us either
    way and its kernels for these tall, narrow problems are no slower.  The setting is global to the
    process (``torch.backends.cuda.preferred_blas_library``); ``get_model`` applies it unless
    ``config.train.dense_blas`` says "default"."""
    torch.backends.cuda.preferred_blas_library("hipblas" if enable else "default")


model_dict = {"sage": HistorySAGE, "rgcn": HistoryRGCN}
graph_type_dict = {"cxg": "CSR_Layer", "dgl": "DGL"}


def get_model(config, table):
    """Model factory with the reference's signature (/root/reference/hiscache/history_model.py:446-470)."""
    mtype = config.train.model.type.lower()
    if str(getattr(config.train, "dense_blas", "rocblas")).lower() != "default":
        prefer_low_latency_gemm()
    if mtype not in model_dict:
        raise NotImplementedError(f"model type {mtype!r}: sage and rgcn are provided")
    if mtype == "rgcn":
        return HistoryRGCN(config.dl.dataset.feature_dim, config.train.model.hidden_dim,
                           config.dl.dataset.num_classes, config.train.model.num_layers,
                           config.train.model.dropout, graph_type_dict[config.train.type.lower()], config,
                           table, num_rel=config.train.model.num_rel,
                           dataset_name=config.dl.dataset.name.lower())
    return model_dict[mtype](config.dl.dataset.feature_dim, config.train.model.hidden_dim,
                             config.dl.dataset.num_classes, config.train.model.num_layers,
                             config.train.model.dropout, graph_type_dict[config.train.type.lower()],
                             config, table)
