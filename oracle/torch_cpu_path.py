"""The hot path spelled with stock PyTorch CPU operators (index_add / scatter semantics).

TEST INFRASTRUCTURE ONLY.  The reference has no CPU implementation; this is its semantics
(/root/reference/src/cpp/src/history_aggr.cu:7-40,127-168; /root/reference/hiscache/history_cache.py:205-221)
written the way a PyTorch user would on a CPU.  Tests use it as a second, independently written
checker of the C oracle.  (The benchmark's CPU baselines are the OpenMP statements in ``hc_cpu_mt.c``,
which run several times faster than this spelling.)
"""
import torch


def edge_rows(ptr, num_node):
    deg = ptr[1:num_node + 1] - ptr[:num_node]
    return torch.repeat_interleave(torch.arange(num_node), deg), deg


def aggr_fwd_row(x, ptr, idx, hmap, hbuf, num_node):
    dst, deg = edge_rows(ptr, num_node)
    E = int(ptr[num_node])
    out = torch.zeros(num_node, x.shape[1], dtype=torch.float32)
    out.index_add_(0, dst, x[idx[:E]].to(torch.float32))
    out = out / deg.clamp(min=1).to(torch.float32)[:, None]
    if hmap is not None:
        is_hist = hmap[:num_node] != -1
        out[is_hist] = hbuf[:num_node][is_hist][:, :x.shape[1]].to(torch.float32)
    return out


def aggr_bwd_row(g, ptr, idx, hmap, n_src, num_node):
    dst, deg = edge_rows(ptr, num_node)
    E = int(ptr[num_node])
    scaled = g / deg.clamp(min=1).to(torch.float32)[:, None]
    ghist = None
    if hmap is not None:
        is_hist = hmap[:num_node] != -1
        scaled = scaled * (~is_hist)[:, None]
        ghist = g * is_hist[:, None]
    gx = torch.zeros(n_src, g.shape[1], dtype=torch.float32)
    gx.index_add_(0, idx[:E], scaled[dst])
    return gx, ghist


def aggr_fwd_src(feat, hist, hmap_src, ptr, idx, num_node):
    dst, deg = edge_rows(ptr, num_node)
    E = int(ptr[num_node])
    src = idx[:E]
    rows = feat[src].to(torch.float32)
    if hmap_src is not None:
        slot = hmap_src[src]
        hit = slot != -1
        rows[hit] = hist[slot[hit]][:, :feat.shape[1]].to(torch.float32)
    out = torch.zeros(num_node, feat.shape[1], dtype=torch.float32)
    out.index_add_(0, dst, rows)
    return out / deg.clamp(min=1).to(torch.float32)[:, None]


def aggr_bwd_src(g, ptr, idx, hmap_src, n_src, num_node):
    """Backward of aggr_fwd_src with respect to ``feat``: substituted sources get a zero row."""
    dst, deg = edge_rows(ptr, num_node)
    E = int(ptr[num_node])
    src = idx[:E]
    scaled = (g / deg.clamp(min=1).to(torch.float32)[:, None])[dst]
    if hmap_src is not None:
        scaled = scaled * (hmap_src[src] == -1)[:, None]
    gx = torch.zeros(n_src, g.shape[1], dtype=torch.float32)
    gx.index_add_(0, src, scaled)
    return gx


def admission(grad, emb, slot, thres, table, header):
    """norm -> mask -> append (history_cache.py:205-221), no ring wrap."""
    norm = grad.norm(dim=1)
    mask = (norm < thres) & (slot == -1)
    n = int(mask.sum())
    table[header:header + n] = emb[mask].to(table.dtype)
    return mask, norm


# --------------------------------------------------------------------------- a whole iteration
def mean_rows(x, ptr, idx, n):
    """Differentiable mean aggregation of the first n rows (index_add over the edge list)."""
    deg = ptr[1:n + 1] - ptr[:n]
    dst = torch.repeat_interleave(torch.arange(n), deg)
    out = torch.zeros(n, x.shape[1], dtype=x.dtype).index_add(0, dst, x[idx[: int(ptr[n])]])
    return out / deg.clamp(min=1).to(x.dtype)[:, None]


def sage_forward(model, ptr, idx, num_node_in_layer, x, slot, cached):
    """HistorySAGE's forward wiring (/root/reference/hiscache/history_model.py:120-153) on the CPU: the layer
    one hop from the seeds takes the cached rows of the hits.  Returns (log-probabilities, that layer's
    aggregation output with retain_grad)."""
    L = model.num_layers
    his = None
    for i, conv in enumerate(model.convs):
        n = int(num_node_in_layer[L - 1 - i])
        agg = mean_rows(x, ptr, idx, n)
        if model.training and i == L - 2:
            agg = torch.where((slot != -1)[:, None], cached, agg)
            if not agg.requires_grad:
                agg.requires_grad_(True)
            agg.retain_grad()
            his = agg
        x = conv.lin_l(agg) + conv.lin_r(x[:n])
        if i < L - 1:
            x = torch.relu(model.bns[i](x))
    return x.log_softmax(dim=-1), his


def ring_state(num_nodes, capacity, hidden, dtype=torch.float32):
    return dict(table=torch.zeros(capacity, hidden, dtype=dtype), f2s=torch.full((num_nodes,), -1, dtype=torch.int64),
                s2f=torch.full((capacity,), -1, dtype=torch.int64), checkin=torch.full((capacity,), -1, dtype=torch.int64),
                header=0)


def sage_iteration(model, opt, batch, feats, state, glb_iter, rate):
    """One training iteration of the plumbing configuration with stock PyTorch CPU operators and the ring
    policy of the reference's history table (/root/reference/hiscache/history_table.py:127-200,
    /root/reference/src/cpp/src/grad_check.cu:6-46): slots and cached rows of the 1-hop nodes, used masks
    (the sequential C statement), masked feature gather, forward, loss, backward, optimizer step, admission of
    the rows whose gradient norm lies below the ``rate`` quantile.  ``batch``: dict of NumPy arrays ptr, idx,
    sub_to_full, num_node_in_layer plus a label tensor y.  Returns the loss."""
    from . import hc_oracle
    ptr, idx = torch.from_numpy(batch["ptr"]), torch.from_numpy(batch["idx"])
    s2f = torch.from_numpy(batch["sub_to_full"])
    nnl = batch["num_node_in_layer"]
    L = model.num_layers
    n_seed, n1, n_all = int(nnl[0]), int(nnl[1]), int(nnl[L])
    ids1 = s2f[:n1]
    slot = state["f2s"][ids1]
    hit = slot != -1
    cached = state["table"][slot.clamp(min=0)].to(torch.float32) * hit[:, None]
    used = hc_oracle.count_history_reconstruct(batch["ptr"], batch["idx"], slot.numpy(), n_all, n_seed, L)
    need = torch.from_numpy(used[0])
    x = feats[s2f] * need[:, None]
    out, his = sage_forward(model, ptr, idx, nnl, x, slot, cached)
    loss = torch.nn.functional.nll_loss(out, batch["y"])
    opt.zero_grad(set_to_none=True)
    loss.backward()
    opt.step()
    with torch.no_grad():
        score = his.grad.norm(dim=1)
        thres = torch.quantile(score, rate)
        mask = (score < thres) & ~hit
        ids = ids1[mask]
        A, cap = ids.numel(), state["table"].shape[0]
        slots = (state["header"] + torch.arange(A)) % cap
        prev = state["s2f"][slots]
        live = prev != -1
        owners = prev[live]
        still = state["f2s"][owners] == slots[live]
        state["f2s"][owners[still]] = -1                      # un-map the previous owners of the slots
        state["table"][slots] = his.detach()[mask].to(state["table"].dtype)
        state["f2s"][ids] = slots
        state["s2f"][slots] = ids
        state["checkin"][slots] = glb_iter
        state["header"] = (state["header"] + A) % cap
    return float(loss.detach())
