import logging

log = logging.getLogger(__name__)


class Config(dict):
    """Minimal stand-in for the OmegaConf tree the reference reads: nested dicts that allow both
    ``cfg.dl.dataset.path`` and ``cfg["dl"]["dataset"]["path"]`` plus ``.get``
    (usage: /root/reference/hiscache/history_cache.py:13-36, history_table.py:12-30)."""

    def __init__(self, mapping=None, **kw):
        super().__init__()
        for k, v in dict(mapping or {}, **kw).items():
            self[k] = Config(v) if isinstance(v, dict) and not isinstance(v, Config) else v

    def __getattr__(self, k):
        try:
            return self[k]
        except KeyError as e:
            raise AttributeError(k) from e

    def __setattr__(self, k, v):
        self[k] = v


def make_config(feature_dim, num_classes, hidden_dim, num_layers, method="grad", rate=0.9,
                staleness_thres=200, limit=0.0, start_history=0, device="cuda:0", path="",
                name="synthetic", model_type="sage", dropout=0.0, train_type="cxg", num_rel=1,
                buffer_size=0, feat_mode="history_uvm", **history_extra):
    """Build the configuration keys the cache, tables and models read, without hydra."""
    hist = dict(method=method, rate=rate, staleness_thres=staleness_thres, limit=limit,
                start_history=start_history, distributed_store=False, store_last_layer=False,
                buffer_size=buffer_size, graph_struct_norm=0)
    hist.update(history_extra)
    return Config({
        "dl": {"dataset": {"feature_dim": feature_dim, "num_classes": num_classes, "path": path,
                           "name": name},
               "num_device": 1, "device": device, "type": train_type,
               "loading": {"feat_mode": feat_mode}},
        "train": {"model": {"type": model_type, "hidden_dim": hidden_dim, "num_layers": num_layers,
                            "dropout": dropout, "num_rel": num_rel},
                  "type": train_type},
        "history": hist,
    })


def quantile_threshold(score, rate):
    """Admission threshold: the ``rate`` quantile of ``score`` with linear interpolation, i.e. what
    ``torch.quantile(score, rate)`` computes (/root/reference/hiscache/history_cache.py:211,
    history_table.py:173), spelled as separately rounded fp32 operations so that CPU and GPU give
    the same bits: with pos = fp32(rate)*fp32(n-1) (an fp32 product, as torch.quantile ranks in the
    data's dtype), lo = floor(pos), w = pos - lo, a = sorted[lo], b = sorted[min(lo+1, n-1)]:
    w < 0.5 -> a + w*(b-a), else b - (b-a)*(1-w).
    Returns a 1-element fp32 tensor on score's device; no host synchronisation."""
    import torch
    n = score.numel()
    if n == 0:
        raise ValueError("quantile of an empty tensor")
    pos = (torch.tensor(float(rate), dtype=torch.float32) * torch.tensor(float(n - 1), dtype=torch.float32))
    lo = min(int(torch.floor(pos).item()), n - 1)
    hi = min(lo + 1, n - 1)
    w = (pos - torch.tensor(float(lo), dtype=torch.float32)).item()
    if score.is_cuda:
        # on the GPU: the two order statistics by a radix select and the interpolation, no sort
        import hiscache_backend
        flat = score.detach().reshape(-1)
        if flat.dtype != torch.float32 or not flat.is_contiguous():
            flat = flat.to(torch.float32).contiguous()
        one_minus_w = (1.0 - torch.tensor(w, dtype=torch.float32)).item()
        return hiscache_backend.quantile_select(flat, lo, hi, w, one_minus_w)
    # host tensors (the CPU tests' spelling of the same rule)
    flat = score.detach().reshape(-1).to(torch.float32)
    srt = torch.sort(flat).values
    a = srt[lo:lo + 1]
    b = srt[hi:hi + 1]
    d = b - a
    if w < 0.5:
        m = d * w
        res = a + m
    else:
        m = d * (1.0 - torch.tensor(w, dtype=torch.float32)).item()
        res = b - m
    # torch.quantile answers NaN when any score is NaN (a sort would rank the NaN last and hide it)
    return torch.where(torch.isnan(flat).any(), torch.full_like(res, float("nan")), res)


def backward_on_this_thread(loss, **kwargs):
    """``loss.backward(**kwargs)`` run by the calling thread instead of autograd's device thread.  The
    nodes of these models are Python functions that enqueue kernels; nothing runs beside them, and the
    hand-over between the two threads costs a sampled-batch iteration 0.06 - 0.1 ms of host time
    (the loop of /root/reference/hiscache/history_trainer.py:176-193 calls ``loss.backward()``)."""
    import torch
    with torch.autograd.set_multithreading_enabled(False):
        loss.backward(**kwargs)
