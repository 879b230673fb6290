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
