"""``hiscache_backend`` -- the operator module of HisCache, for MI355X.

Drop-in for the reference's pybind11 module of the same name
(/root/reference/src/cpp/python_bindings/binding.cpp:9-24): the six in-scope
callables keep their names and positional signatures

    aggr_forward_history, aggr_forward_history_edge_value, record_history,
    count_history_reconstruct, get_graph_structure_score, count_num

but run hand-written gfx950 kernels from ``libhiscache_hip.so`` through its C
ABI (ctypes; raw device pointers, sizes, dtype enums, the current HIP stream).
``p2psend`` / ``p2psend_gentensor`` (multi-GPU) are not provided.

Beyond the reference's set: ``aggr_forward_source_history`` (per-source substitution),
``build_transpose``, ``row_scores``, ``grad_check`` / ``cache_append`` (fused admission), ``evict``,
``gather_rows`` / ``lookup``, ``typed_csr`` / ``edge_types_by_ranges`` (relational blocks),
``sample_layers`` (device sampler), ``bias_bn_relu`` (a hidden layer's epilogue) and ``check_csr`` (input
validation).

There is no CPU or PyTorch fallback: if the shared library is missing or a
tensor is not on a GPU, the call raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# HISCACHE_HIP_LIB overrides the location of the built library (default: next to this file)
LIB_PATH = os.environ.get("HISCACHE_HIP_LIB") or os.path.join(_HERE, "libhiscache_hip.so")

# enums of include/hiscache_hip.h
HC_F32, HC_F16, HC_BF16 = 0, 1, 2
SUBST_ROW, SUBST_SRC = 0, 1
NORM_L2, NORM_L1 = 0, 1
CMP_LT, CMP_NOT_GT = 0, 1
GRAD_CHECK_STATIC_MAX_ROWS = 1 << 24   # HC_GRAD_CHECK_STATIC_MAX_ROWS

_DTYPES = {torch.float32: HC_F32, torch.float16: HC_F16, torch.bfloat16: HC_BF16}

_c_i64 = ctypes.c_int64
_c_p = ctypes.c_void_p
_c_int = ctypes.c_int
_c_sz = ctypes.c_size_t

# name -> (restype, argtypes): the full export list of include/hiscache_hip.h
_SIGNATURES = {
    "hc_version": (ctypes.c_char_p, []),
    "hc_strerror": (ctypes.c_char_p, [_c_int]),
    "hc_device_count": (_c_int, []),
    "hc_aggr_fwd_workspace_bytes": (_c_sz, [_c_int, _c_i64, _c_i64, _c_i64]),
    "hc_aggr_fwd": (_c_int, [_c_int, _c_p, _c_p, _c_p, _c_int, _c_p, _c_p, _c_int, _c_i64, _c_p, _c_i64,
                             _c_p, _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p]),
    "hc_aggr_fwd_long_row_edges": (_c_i64, [_c_i64, _c_int]),
    "hc_transpose_workspace_bytes": (_c_sz, [_c_i64, _c_i64, _c_i64]),
    "hc_build_transpose": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_p,
                                    _c_sz, _c_p]),
    "hc_transpose_dev_workspace_bytes": (_c_sz, [_c_i64, _c_i64]),
    "hc_build_transpose_dev": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p,
                                        _c_sz, _c_p]),
    "hc_build_transpose_dev_deg": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p,
                                            _c_p, _c_sz, _c_p]),
    "hc_aggr_bwd_workspace_bytes": (_c_sz, [_c_i64, _c_i64]),
    "hc_aggr_bwd_chunk_edges": (_c_i64, [_c_i64]),
    "hc_aggr_bwd": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_i64, _c_p,
                             _c_p, _c_i64, _c_p, _c_i64, _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p]),
    "hc_aggr_bwd_batch_view": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_i64,
                                        _c_i64, _c_p, _c_sz, _c_p]),
    "hc_aggr_bwd_batch_view_typed": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_int, _c_p, _c_p, _c_p, _c_i64,
                                              _c_i64, _c_i64, _c_p]),
    "hc_load_mask": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_p]),
    "hc_count_history": (_c_int, [_c_p, _c_p, _c_p, _c_i64, _c_p, _c_i64, _c_i64, _c_i64, _c_int, _c_p]),
    "hc_row_scores": (_c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_int, _c_p]),
    "hc_quantile_max_scores": (_c_i64, []),
    "hc_quantile_threshold": (_c_int, [_c_p, _c_i64, _c_i64, _c_i64, ctypes.c_float, ctypes.c_float, _c_p, _c_p]),
    "hc_quantile_workspace_bytes": (_c_sz, [_c_i64]),
    "hc_quantile_threshold_ws": (_c_int, [_c_p, _c_i64, _c_i64, _c_i64, ctypes.c_float, ctypes.c_float, _c_p, _c_p,
                                          _c_sz, _c_p]),
    "hc_grad_check_workspace_bytes": (_c_sz, [_c_i64]),
    "hc_grad_check": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, ctypes.c_int32, _c_int,
                               _c_int, _c_p, _c_p, _c_p, _c_p, _c_int, _c_i64, _c_p, _c_p, _c_p, _c_p,
                               _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p]),
    "hc_grad_check_static": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, ctypes.c_int32, _c_int,
                                      _c_int, _c_p, _c_p, _c_p, _c_p, _c_int, _c_i64, _c_p, _c_p, _c_p, _c_p,
                                      _c_i64, _c_i64, _c_i64, _c_p]),
    "hc_record_history": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
                                   _c_i64, _c_i64, _c_i64, _c_i64, _c_p, _c_sz, _c_p]),
    "hc_cache_append": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_p,
                                 _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_sz, _c_p]),
    "hc_count_num": (_c_int, [_c_p, _c_i64, _c_i64, _c_p, _c_p]),
    "hc_structure_score": (_c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_int, _c_p, _c_p, _c_p]),
    "hc_gather_rows": (_c_int, [_c_p, _c_int, _c_i64, _c_p, _c_p, _c_p, _c_int, _c_int, _c_i64, _c_i64, _c_p]),
    "hc_stream_create_cu_limited": (_c_int, [_c_int, _c_p]),
    "hc_stream_destroy": (_c_int, [_c_p]),
    "hc_gather_rows_hot": (_c_int, [_c_p, _c_int, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_int, _c_p, _c_i64, _c_i64,
                                    _c_p]),
    "hc_gather_rows_flagged": (_c_int, [_c_p, _c_int, _c_i64, _c_p, _c_p, _c_p, _c_int, _c_i64, _c_i64, _c_p]),
    "hc_fixup_rows": (_c_int, [_c_p, _c_int, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_int, _c_i64, _c_i64, _c_p]),
    "hc_lookup": (_c_int, [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_p]),
    "hc_lookup_dev": (_c_int, [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p]),
    "hc_ring_lookup": (_c_int, [_c_p, _c_i64, _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_int, _c_i64, _c_i64, _c_p, _c_p,
                                _c_i64, _c_p]),
    "hc_check_csr": (_c_int, [_c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_p, _c_p]),
    "hc_evict": (_c_int, [_c_p, _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_p]),
    "hc_sample_capacity": (_c_int, [_c_i64, _c_p, _c_int, _c_i64, _c_p, _c_p, _c_p]),
    "hc_sample_workspace_bytes": (_c_sz, [_c_i64, _c_p, _c_int, _c_i64]),
    "hc_sample_map_init": (_c_int, [_c_p, _c_i64, _c_p]),
    "hc_sample_layers": (_c_int, [_c_p, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_int, ctypes.c_uint64, _c_p, _c_p,
                                  _c_p, _c_p, _c_p, _c_p, _c_sz, _c_p]),
    "hc_sample_layers_seed_at": (_c_int, [_c_p, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_int, _c_p, _c_p, _c_p,
                                          _c_p, _c_p, _c_p, _c_p, _c_sz, _c_p]),
    "hc_bn_relu_workspace_bytes": (_c_sz, [_c_i64, _c_i64]),
    "hc_bn_relu_fwd": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, ctypes.c_float, ctypes.c_float, _c_p,
                                _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_sz, _c_p, _c_p]),
    "hc_bn_relu_bwd": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64,
                                _c_p, _c_sz, _c_p, _c_p]),
    "hc_weight_grad_workspace_bytes": (_c_sz, [_c_i64, _c_i64, _c_i64, _c_int]),
    "hc_weight_grad": (_c_int, [_c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_p, _c_p, _c_p, _c_sz, _c_p]),
    "hc_stage_arrays": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_p, _c_p, _c_int, _c_p]),
    "hc_ring_lookup_dev": (_c_int, [_c_p, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_p, _c_int, _c_i64, _c_i64, _c_p,
                                    _c_p, _c_i64, _c_p]),
    "hc_grad_check_dev": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, ctypes.c_int32, _c_int,
                                   _c_int, _c_p, _c_p, _c_p, _c_p, _c_int, _c_i64, _c_p, _c_p, _c_p, _c_p,
                                   _c_p, _c_i64, _c_i64, _c_p, _c_sz, _c_p]),
    "hc_quantile_threshold_dev": (_c_int, [_c_p, _c_p, _c_i64, ctypes.c_float, _c_p, _c_p]),
    "hc_bn_relu_fwd_dev": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, ctypes.c_float, ctypes.c_float, _c_p,
                                    _c_p, _c_p, _c_i64, _c_i64, _c_p, _c_p, _c_sz, _c_p, _c_p]),
    "hc_bn_relu_bwd_dev": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64,
                                    _c_p, _c_p, _c_sz, _c_p, _c_p]),
    "hc_typed_csr_workspace_bytes": (_c_sz, [_c_i64, _c_int]),
    "hc_edge_types_by_ranges": (_c_int, [_c_p, _c_p, _c_p, _c_i64, _c_p, _c_int, _c_p, _c_p, _c_i64, _c_i64, _c_p]),
    "hc_typed_csr": (_c_int, [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64, _c_int, _c_p, _c_p, _c_p, _c_p,
                              _c_p, _c_p, _c_sz, _c_p, _c_p]),
}

_lib_handle = None

def load_library():
    """Load ``libhiscache_hip.so`` and bind every export.  Raises if it is not built."""
    global _lib_handle
    if _lib_handle is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}` "
                "(there is no fallback path)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib_handle = lib
    return _lib_handle


def exported_symbols():
    return sorted(_SIGNATURES)


def _check(rc, what):
    if rc != 0:
        msg = load_library().hc_strerror(rc).decode()
        if rc in (1, 2, 4, 5):
            raise ValueError(f"{what}: {msg}")
        raise RuntimeError(f"{what}: {msg}")


def _raw_stream(device_index=None):
    """Handle of the current HIP stream of a device (default: the current device) as an integer.
    torch's private accessor returns it directly (0.3 us); building a torch.cuda.Stream object for it costs
    2.7 us, and every call of this module asks at least once."""
    if device_index is None:
        device_index = torch.cuda.current_device()
    get = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if get is not None:
        return int(get(device_index))
    return int(torch.cuda.current_stream(device_index).cuda_stream)


def _stream():
    return _c_p(_raw_stream())


def _ptr(t):
    if t is None:
        return _c_p(None)
    return _c_p(t.data_ptr())


def _dev(t, name, dtype=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); this module has no CPU path")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t


def _float_dtype(t, name):
    if t.dtype not in _DTYPES:
        raise ValueError(f"{name} must be float32, float16 or bfloat16, got {t.dtype}")
    return _DTYPES[t.dtype]


def _empty(t):
    return t is None or t.numel() == 0


# Scratch memory of the calls.  Every entry point's workspace is dead when its kernels have run, and calls
# issued on one stream run in order, so the calls of a stream share one buffer that grows to the largest
# request seen (up to _WS_KEEP_BYTES; larger requests, and calls on a capturing stream, whose buffer must
# stay alive with the graph, get a buffer of their own).  Sampled batches change every size at every
# iteration; without this each call paid an allocator look-up, and a device allocation when it missed.
_WS_KEEP_BYTES = 64 << 20
_ws_cache = {}


def _workspace(nbytes, device):
    nbytes = max(int(nbytes), 256)
    if nbytes > _WS_KEEP_BYTES or torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    key = (device.index, _raw_stream(device.index))
    buf = _ws_cache.get(key)
    if buf is None or buf.numel() < nbytes:
        size = 1 << 20
        while size < nbytes:
            size <<= 1
        buf = _ws_cache[key] = torch.empty(size, dtype=torch.uint8, device=device)
    return buf


def release_workspaces():
    """Drop the per-stream scratch buffers (they are allocated again on demand)."""
    _ws_cache.clear()


# With HISCACHE_CHECK_INPUTS=1 every aggregation call first checks its CSR block on the device
# (one extra launch and a synchronisation: for debugging, the kernels themselves trust their indices).
CHECK_INPUTS = os.environ.get("HISCACHE_CHECK_INPUTS", "0") not in ("", "0")


def check_csr(ptr, idx, num_node, n_src):
    """Raise ValueError if the first ``num_node`` rows of (ptr, idx) are not a valid CSR block over
    ``n_src`` sources: offsets must not decrease and must stay inside ``idx``, ids inside [0, n_src)."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    R = int(num_node)
    if R < 0 or R > ptr.numel() - 1:
        raise ValueError("num_node exceeds the rows of ptr")
    report = torch.empty(4, dtype=torch.int64, device=ptr.device)
    _check(lib.hc_check_csr(_ptr(ptr), _ptr(idx), R, idx.numel(), int(n_src), _ptr(report), _stream()),
           "hc_check_csr")
    bad = report.tolist()
    if any(bad[:3]):
        raise ValueError(f"invalid CSR block: {bad[0]} rows end before they start, {bad[1]} offsets outside "
                         f"[0, {idx.numel()}], {bad[2]} neighbour ids outside [0, {int(n_src)})")


# ----------------------------------------------------------------------------- raw launchers
def _aggr_fwd(mode, ptr, idx, x, hmap, hbuf, hsize, edge_value, num_node):
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    _dev(x, "input")
    R = int(num_node) if num_node else ptr.numel() - 1
    if R < 0 or R > ptr.numel() - 1:
        raise ValueError("num_node exceeds the rows of ptr")
    n_head = 1
    if edge_value is not None:
        _dev(edge_value, "edge_value", torch.float32)
        if edge_value.dim() == 2:
            n_head = edge_value.shape[1]
            if x.dim() != 3 or x.shape[1] != n_head:
                raise ValueError("multi-head edge_value needs input of shape [N, H, F] with the same H")
        elif edge_value.dim() != 1:
            raise ValueError("edge_value must be [E] or [E, H]")
    F = x.shape[-1]
    n_src = x.shape[0]
    if hmap is not None:
        _dev(hmap, "history_map", torch.int64)
        _dev(hbuf, "history_buffer")
        need = R if mode == SUBST_ROW else n_src
        if hmap.numel() < need:
            raise ValueError(f"history_map has {hmap.numel()} entries, needs {need}")
        if mode == SUBST_ROW and hbuf.numel() < R * hsize:
            raise ValueError("history_buffer is smaller than num_node x history_size")
    if CHECK_INPUTS:
        check_csr(ptr, idx, R, n_src)
    out_shape = (R, F) if n_head == 1 and x.dim() == 2 else (R, n_head, F)
    out = torch.empty(out_shape, dtype=torch.float32, device=x.device)
    # scratch for the long-row list (large blocks only: the library reports 0 bytes otherwise)
    ws_bytes = int(lib.hc_aggr_fwd_workspace_bytes(mode, R, idx.numel(), n_src)) if n_head == 1 else 0
    ws = _workspace(ws_bytes, x.device) if ws_bytes > 0 else None
    rc = lib.hc_aggr_fwd(mode, _ptr(ptr), _ptr(idx), _ptr(x), _float_dtype(x, "input"),
                         _ptr(hmap), _ptr(hbuf), _float_dtype(hbuf, "history_buffer") if hmap is not None else 0,
                         int(hsize), _ptr(edge_value), n_head, _ptr(out), R, F, n_src, _ptr(ws), ws_bytes,
                         _stream())
    _check(rc, "hc_aggr_fwd")
    return out


def build_transpose(ptr, idx, history_map_row, num_node, n_src, num_edge=None, want_edges=True,
                    history_map_src=None):
    """Stable CSC view of the first ``num_node`` rows: returns (ptrT, rowT, edgeT).

    ``num_edge`` bounds the edge slots that are sorted (default: all of ``idx``).  With
    ``want_edges=False`` (enough for the mean aggregation) edgeT is None and the build is cheaper.
    Edges of rows flagged by ``history_map_row`` and edges whose source is flagged by
    ``history_map_src`` (per-source substitution) are left out."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    R = int(num_node) if num_node else ptr.numel() - 1
    E = int(num_edge) if num_edge is not None else idx.numel()
    E = min(E, idx.numel())
    dev = ptr.device
    ptrT = torch.empty(n_src + 1, dtype=torch.int64, device=dev)
    rowT = torch.empty(max(E, 1), dtype=torch.int32, device=dev)
    edgeT = torch.empty(max(E, 1), dtype=torch.int32, device=dev) if want_edges else None
    nbytes = lib.hc_transpose_workspace_bytes(R, E, n_src)
    if nbytes == 0:
        raise RuntimeError("hc_transpose_workspace_bytes failed (no usable GPU?)")
    ws = _workspace(nbytes, dev)
    hm = None if _empty(history_map_row) else _dev(history_map_row, "history_map", torch.int64)
    hs = None if _empty(history_map_src) else _dev(history_map_src, "source_history_map", torch.int64)
    if hs is not None and hs.numel() < n_src:
        raise ValueError("source_history_map is shorter than n_src")
    if hm is not None and hm.numel() < R:
        raise ValueError("history_map is shorter than num_node")
    rc = lib.hc_build_transpose(_ptr(ptr), _ptr(idx), _ptr(hm), _ptr(hs), R, E, n_src, _ptr(ptrT), _ptr(rowT),
                                _ptr(edgeT), _ptr(ws), ws.numel(), _stream())
    _check(rc, "hc_build_transpose")
    return ptrT, rowT, edgeT


def _aggr_bwd(ptr, idx, tr, g, hmap, edge_value, x, want_edge_grad, hbuf_shape, hsize, num_node, n_src,
              want_hist_grad=True):
    """Gradient of the aggregation: (grad_input, grad_history_buffer or None, edge_grad or None).
    ``want_hist_grad=False`` skips the history buffer's gradient (a full-size write that a cached
    embedding without ``requires_grad`` has no use for)."""
    lib = load_library()
    ptrT, rowT, edgeT = tr
    g = _dev(g.contiguous(), "grad_output", torch.float32)
    R = int(num_node)
    F = g.shape[-1]
    n_head = g.shape[1] if g.dim() == 3 else 1
    dev = g.device
    gshape = (n_src, F) if g.dim() == 2 else (n_src, n_head, F)
    grad_x = torch.empty(gshape, dtype=torch.float32, device=dev)
    grad_h = None
    if hmap is not None and want_hist_grad:
        grad_h = torch.empty(hbuf_shape, dtype=torch.float32, device=dev)
        if grad_h.numel() != R * hsize:
            # history buffers longer than num_node rows: only the first num_node rows get gradient
            grad_h.zero_()
    edge_grad = None
    if want_edge_grad:
        edge_grad = torch.empty_like(edge_value)
    E_total = rowT.numel()
    if edge_value is not None:
        E_total = max(E_total, edge_value.shape[0]) if edge_grad is None else edge_value.shape[0]
    nbytes = lib.hc_aggr_bwd_workspace_bytes(rowT.numel(), F) if edge_value is None and n_head == 1 else 0
    ws = _workspace(nbytes, dev) if nbytes else None
    rc = lib.hc_aggr_bwd(_ptr(ptr), _ptr(idx), _ptr(ptrT), _ptr(rowT), _ptr(edgeT), _ptr(g), _ptr(hmap),
                         _ptr(edge_value), _ptr(x) if want_edge_grad else _c_p(None),
                         _float_dtype(x, "input") if want_edge_grad else 0, n_head, _ptr(grad_x),
                         _ptr(grad_h), int(hsize), _ptr(edge_grad), E_total, R, F, n_src, _ptr(ws),
                         ws.numel() if ws is not None else 0, _stream())
    _check(rc, "hc_aggr_bwd")
    return grad_x, grad_h, edge_grad


class BatchView:
    """One transposed view of a whole mini-batch CSR, shared by the layers of the batch: ``ptrT`` over
    all ``n_src`` nodes of the batch, ``rowT`` (and ``edgeT`` when built) over the edges of its first
    ``rows`` rows.  A layer that owns the first R <= rows rows and the first n <= n_src sources uses a
    prefix of ``ptrT``; edges of other rows are stepped over in backward.  ``num_edge`` bounds the
    entries of ``rowT`` that hold edges."""
    __slots__ = ("ptrT", "rowT", "edgeT", "rows", "n_src", "num_edge", "max_in_degree")

    def __init__(self, ptrT, rowT, edgeT, rows, n_src, num_edge, max_in_degree=None):
        self.ptrT, self.rowT, self.edgeT = ptrT, rowT, edgeT
        self.rows, self.n_src, self.num_edge = int(rows), int(n_src), int(num_edge)
        # the largest number of edges that one node of the batch has in the view, when whoever made the batch
        # knows it (None: unknown).  A view without a source above the backward's chunk length needs neither
        # the chunk sums nor the launch that combines them.
        self.max_in_degree = None if max_in_degree is None else int(max_in_degree)

    def covers(self, num_node, n_src):
        return int(num_node) <= self.rows and int(n_src) <= self.n_src

    def record_stream(self, stream):
        for t in (self.ptrT, self.rowT, self.edgeT):
            if t is not None:
                t.record_stream(stream)


def build_batch_view(ptr, idx, num_node, n_src, num_edge=None, want_edges=False):
    """The shared view of a mini-batch: the stable transposed view of the first ``num_node`` rows of
    (ptr, idx) -- all rows of the batch's CSR -- over ``n_src`` nodes, with nothing left out.  A loader
    builds it once per batch, ahead of the training step (the device sampler does, with
    ``emit_view=True``)."""
    R = int(num_node) if num_node else ptr.numel() - 1
    E = idx.numel() if num_edge is None else min(int(num_edge), idx.numel())
    ptrT, rowT, edgeT = build_transpose(ptr, idx, None, R, int(n_src), num_edge=E, want_edges=want_edges)
    return BatchView(ptrT, rowT, edgeT, R, n_src, E)


def check_batch_view(view, n_src):
    """Raise ValueError if the first ``n_src`` columns of a batch's transposed view are not valid: column offsets
    must not decrease and must stay inside ``rowT``, rows inside [0, view.rows) (and edge slots, where the view
    holds them, inside [0, view.num_edge))."""
    if view.rowT.dtype != torch.int32:
        raise ValueError("rowT must be int32")
    check_csr(view.ptrT, view.rowT.to(torch.int64), n_src, view.rows)
    if view.edgeT is not None:
        check_csr(view.ptrT, view.edgeT.to(torch.int64), n_src, max(view.num_edge, 1))


def _aggr_bwd_batch_view(ptr, view, g, hmap, hbuf_shape, hsize, num_node, n_src, want_hist_grad=True):
    """Gradient of the mean aggregation over the batch's shared view: (grad_input, grad_history or None)."""
    lib = load_library()
    g = _dev(g.contiguous(), "grad_output", torch.float32)
    if g.dim() != 2:
        raise ValueError("the shared view serves the plain mean: grad_output must be [num_node, F]")
    R, F = int(num_node), g.shape[1]
    if not view.covers(R, n_src):
        raise ValueError(f"the batch view covers {view.rows} rows / {view.n_src} sources, "
                         f"the layer has {R} / {n_src}")
    if g.shape[0] < R or (hmap is not None and hmap.numel() < R):
        raise ValueError("grad_output or history_map is shorter than num_node")
    if CHECK_INPUTS:
        check_batch_view(view, n_src)
    dev = g.device
    grad_x = torch.empty((n_src, F), dtype=torch.float32, device=dev)
    grad_h = None
    if hmap is not None and want_hist_grad:
        grad_h = torch.empty(hbuf_shape, dtype=torch.float32, device=dev)
        if grad_h.numel() != R * hsize:
            grad_h.zero_()
    chunk = bwd_chunk_edges(F)
    hubless = view.max_in_degree is not None and (chunk == 0 or view.max_in_degree <= chunk)
    nbytes = 0 if hubless else lib.hc_aggr_bwd_workspace_bytes(view.num_edge, F)
    ws = _workspace(nbytes, dev) if nbytes else None
    rc = lib.hc_aggr_bwd_batch_view(_ptr(ptr), _ptr(view.ptrT), _ptr(view.rowT), _ptr(g), _ptr(hmap),
                                    _ptr(grad_x), _ptr(grad_h), int(hsize), view.num_edge, R, F, int(n_src),
                                    _ptr(ws), ws.numel() if ws is not None else 0, _stream())
    _check(rc, "hc_aggr_bwd_batch_view")
    return grad_x, grad_h


def typed_batch_view_supported(view, num_node, n_src, feature_width):
    """Can ``_aggr_bwd_typed_batch_view`` serve this layer (view with edge slots that covers it, fast width)?"""
    return (view is not None and view.edgeT is not None and view.covers(num_node, n_src)
            and bwd_chunk_edges(feature_width) > 0)


def _aggr_bwd_typed_batch_view(ptr, view, edge_types, num_rel, used_mask, g, num_node, n_src):
    """Input gradient of the relational layer over the batch's shared view: g is the gradient of the
    (row, relation) groups' sums, [num_node * num_rel, F]."""
    lib = load_library()
    g = _dev(g.contiguous(), "grad_output", torch.float32)
    _dev(edge_types, "edge_types", torch.int64)
    R, K, F = int(num_node), int(num_rel), g.shape[-1]
    if g.dim() != 2 or g.shape[0] < R * K:
        raise ValueError("grad_output must be [num_node * num_rel, F]")
    if not view.covers(R, n_src) or view.edgeT is None:
        raise ValueError("the batch view does not cover this layer, or was built without edge slots")
    if used_mask is not None:
        used_mask = _dev(used_mask, "used_mask")
        if used_mask.element_size() != 1 or used_mask.numel() < n_src:
            raise ValueError("used_mask must hold one byte per source")
    if CHECK_INPUTS:
        check_batch_view(view, n_src)
    E = min(int(edge_types.numel()), view.num_edge)
    grad_x = torch.empty((int(n_src), F), dtype=torch.float32, device=g.device)
    rc = lib.hc_aggr_bwd_batch_view_typed(_ptr(ptr), _ptr(view.ptrT), _ptr(view.rowT), _ptr(view.edgeT),
                                          _ptr(edge_types), E, K, _ptr(used_mask), _ptr(g), _ptr(grad_x), R, F,
                                          int(n_src), _stream())
    _check(rc, "hc_aggr_bwd_batch_view_typed")
    return grad_x


class _AggrHistory(torch.autograd.Function):
    """Counterpart of AggrHistoryFunction / AggrHistoryEdgeValueFunction
    (/root/reference/src/cpp/src/history_aggr.cu:475-596).  Tensor references are kept on the
    context (the reference keeps raw addresses, :406-408)."""

    @staticmethod
    def forward(ctx, x, ptr, idx, edge_value, hmap, hbuf, hsize, num_node, mode, num_edge=None, view=None):
        R = int(num_node) if num_node else ptr.numel() - 1
        out = _aggr_fwd(mode, ptr, idx, x, hmap, hbuf, hsize, edge_value, R)
        ctx.hc = (ptr, idx, hmap, hsize, R, mode, None if hbuf is None else tuple(hbuf.shape))
        # edge slots the first R rows can reach, when the caller knows it (a layer of a shared CSR owns a
        # prefix of idx): the transposed view then sorts that prefix only
        ctx.num_edge = num_edge
        # the batch's shared transposed view (plain mean with per-row substitution only)
        ctx.view = view if (edge_value is None and mode == SUBST_ROW and view is not None
                            and view.covers(R, x.shape[0]) and x.dim() == 2) else None
        ctx.hdtype = None if hbuf is None else hbuf.dtype
        ctx.save_for_backward(x, edge_value if edge_value is not None else x.new_empty(0))
        ctx.has_ev = edge_value is not None
        return out

    @staticmethod
    def backward(ctx, g):
        ptr, idx, hmap, hsize, R, mode, hshape = ctx.hc
        x, ev = ctx.saved_tensors
        ev = ev if ctx.has_ev else None
        n_src = x.shape[0]
        row_map = hmap if mode == SUBST_ROW else None
        want_x = ctx.needs_input_grad[0]
        want_eg = ev is not None and ctx.needs_input_grad[3]
        want_h = row_map is not None and ctx.needs_input_grad[5]
        if not want_x and not want_eg:
            # raw features at the input layer: nothing flows further back, so the transposed view
            # and the gather are skipped; the history buffer's gradient is a masked copy of g
            grad_h = None
            if want_h:
                g2 = g.contiguous()
                if g2.dim() == 3 and hsize == g2.shape[-1]:
                    g2 = g2.sum(1)
                grad_h = torch.zeros(hshape, dtype=torch.float32, device=g.device)
                flat = g2.reshape(R, -1)
                hit = (row_map[:R] != -1).unsqueeze(1)
                grad_h.view(-1, hsize)[:R, :flat.shape[1]] = torch.where(hit, flat, torch.zeros_like(flat))
            return None, None, None, None, None, grad_h, None, None, None, None, None
        if ctx.view is not None:
            grad_x, grad_h = _aggr_bwd_batch_view(ptr, ctx.view, g, row_map, hshape, hsize, R, n_src,
                                                  want_hist_grad=want_h)
            if grad_x.dtype != x.dtype:
                grad_x = grad_x.to(x.dtype)
            if grad_h is not None and grad_h.dtype != ctx.hdtype:
                grad_h = grad_h.to(ctx.hdtype)
            return grad_x, None, None, None, None, grad_h, None, None, None, None, None
        # The transposed view is built here, on the stream backward runs on.  Building it during the
        # forward pass on a side stream was measured and dropped: concurrent with the bandwidth-bound
        # forward it finishes no earlier (9.15 against 9.09 ms for forward + backward on a 20 M-edge
        # block), and on sampled mini-batches the stream switch costs the host more than the build
        # costs the GPU.
        src_map = hmap if mode == SUBST_SRC else None
        want_table = src_map is not None and ctx.needs_input_grad[5]
        # Per-source substitution: a substituted source passes nothing to input[s] (that row was never
        # read).  When the table needs no gradient those edges are left out of the view; when it does,
        # every source is summed and the rows of substituted sources are moved to the table's gradient.
        num_edge = ctx.num_edge
        tr = build_transpose(ptr, idx, row_map, R, n_src, num_edge=num_edge, want_edges=ev is not None,
                             history_map_src=None if want_table else src_map)
        grad_x, grad_h, edge_grad = _aggr_bwd(ptr, idx, tr, g, row_map, ev, x, want_eg, hshape, hsize, R,
                                              n_src, want_hist_grad=want_h)
        if want_table:
            sub = src_map[:n_src] != -1
            grad_h = torch.zeros(hshape, dtype=torch.float32, device=g.device)
            grad_h.view(-1, hsize)[:, :grad_x.shape[-1]].index_add_(0, src_map[:n_src][sub], grad_x[sub])
            grad_x = grad_x.masked_fill(sub.unsqueeze(1), 0.0)
        elif mode == SUBST_SRC or not want_h:
            grad_h = None
        if grad_x.dtype != x.dtype:
            grad_x = grad_x.to(x.dtype)
        if grad_h is not None and grad_h.dtype != ctx.hdtype:
            grad_h = grad_h.to(ctx.hdtype)
        return (grad_x if want_x else None), None, None, edge_grad, None, grad_h, None, None, None, None, None


def _norm_history(history_map, history_buffer, history_size):
    # an empty buffer: no row can be substituted (the reference's no-cache mode hands over a map of -1 and an
    # empty tensor, /root/reference/hiscache/history_cache.py:291-294, and its kernel then reads no history row)
    if history_size == 0 or _empty(history_map) or _empty(history_buffer):
        return None, None, 0
    return history_map, history_buffer, int(history_size)


# ----------------------------------------------------------------------------- reference API
def aggr_forward_history(input, ptr, idx, history_map, history_buffer, history_size, num_node, num_edge=None,
                         view=None):
    """Mean aggregation with history substitution; same positional signature as the reference
    (/root/reference/src/cpp/include/history_aggr.h:34-37).  ``history_size == 0`` or an
    empty ``history_map`` gives the plain mean (the reference exits there, history_aggr.cu:440-441).
    The result always requires grad (history_aggr.cu:604).  ``num_edge`` (optional, beyond the
    reference) is an upper bound of ptr[num_node] for callers that know it -- a layer of a shared
    mini-batch CSR owns a prefix of ``idx`` -- so that backward looks at that prefix only.  ``view``
    (optional, a ``BatchView``) is the batch's shared transposed view: backward then builds none."""
    hmap, hbuf, hsize = _norm_history(history_map, history_buffer, history_size)
    out = _AggrHistory.apply(input, ptr, idx, None, hmap, hbuf, hsize, num_node, SUBST_ROW, num_edge, view)
    if not out.requires_grad:
        out.requires_grad_(True)
    return out


def aggr_forward_history_edge_value(input, ptr, idx, edge_value, history_map, history_buffer,
                                    history_size, num_node):
    """Weighted (and multi-head) aggregation; same signature as the reference
    (/root/reference/src/cpp/include/history_aggr.h:39-42).  An empty ``edge_value`` falls
    back to the mean op, as the reference's dispatch does (history_aggr.cu:439)."""
    if _empty(edge_value):
        return aggr_forward_history(input, ptr, idx, history_map, history_buffer, history_size, num_node)
    hmap, hbuf, hsize = _norm_history(history_map, history_buffer, history_size)
    out = _AggrHistory.apply(input, ptr, idx, edge_value, hmap, hbuf, hsize, num_node, SUBST_ROW)
    if not out.requires_grad:
        out.requires_grad_(True)
    return out


def aggr_forward_source_history(input, ptr, idx, source_history_map, history_table, num_node=0):
    """Extension: per-SOURCE substitution.  Neighbour j is read from
    ``history_table[source_history_map[idx[j]]]`` when the map entry is not -1, else from
    ``input[idx[j]]``.  Backward: ``input`` rows of substituted sources get a zero gradient (they
    were not read); their share goes to ``history_table``'s gradient when it requires one."""
    hsize = 0 if _empty(source_history_map) else history_table.shape[-1]
    hmap, hbuf, hsize = _norm_history(source_history_map, history_table, hsize)
    return _AggrHistory.apply(input, ptr, idx, None, hmap, hbuf, hsize, num_node, SUBST_SRC)


def count_history_reconstruct(ptr, idx, history_maps, num_node, num_seed, num_layer):
    """Per-level "still needed" masks; same signature and result layout as the reference
    (/root/reference/src/cpp/include/grad_check.h:18-20): a list of num_layer+1 bool tensors
    of size num_node, [0] = raw-feature level, [num_layer] = seed level."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    hm = None if _empty(history_maps) else _dev(history_maps, "history_maps", torch.int64)
    L = int(num_layer)
    masks = torch.empty((L + 1, int(num_node)), dtype=torch.uint8, device=ptr.device)
    rc = lib.hc_count_history(_ptr(ptr), _ptr(idx), _ptr(hm), 0 if hm is None else hm.numel(), _ptr(masks),
                              ptr.numel() - 1, int(num_node), int(num_seed), L, _stream())
    _check(rc, "hc_count_history")
    masks = masks.view(torch.bool)
    return [masks[i] for i in range(L + 1)]


def record_history(buffer_new, buffer_all, used_mask, sub_to_full, sub_to_history, history_to_full,
                   full_to_history, header, score, thres, checkin_iter, glb_iter):
    """Ring-buffer admission on precomputed scores; same signature as the reference
    (/root/reference/src/cpp/include/grad_check.h:12-16).  In place on ``buffer_all``,
    ``history_to_full``, ``full_to_history``, ``header`` and ``checkin_iter``.  Slots are handed
    out in row order (the reference: atomic arrival order)."""
    lib = load_library()
    _dev(buffer_new, "buffer_new", torch.float32)
    _dev(buffer_all, "buffer_all", torch.float32)
    M = buffer_new.shape[0]
    hs = buffer_all.shape[1] if buffer_all.dim() == 2 else buffer_new.shape[1]
    if buffer_new.dim() != 2 or buffer_new.shape[1] != hs:
        raise ValueError("buffer_new must be [M, history_size]")
    um = _dev(used_mask, "used_mask")
    if um.dtype not in (torch.bool, torch.uint8):
        raise ValueError("used_mask must be bool")
    for t, n in ((sub_to_full, "sub_to_full"), (sub_to_history, "sub_to_history"),
                 (history_to_full, "history_to_full"), (full_to_history, "full_to_history"),
                 (header, "header"), (checkin_iter, "checkin_iter")):
        _dev(t, n, torch.int64)
    _dev(score, "score", torch.float32)
    thres = _dev(thres.reshape(1).contiguous(), "thres", torch.float32)
    if min(um.numel(), sub_to_full.numel(), sub_to_history.numel(), score.numel()) < M:
        raise ValueError("per-row arguments are shorter than buffer_new")
    nbytes = lib.hc_grad_check_workspace_bytes(M) + (M + 255) // 256 * 256
    ws = _workspace(nbytes, buffer_new.device)
    rc = lib.hc_record_history(_ptr(buffer_new), _ptr(buffer_all), _ptr(um), _ptr(sub_to_full),
                               _ptr(sub_to_history), _ptr(history_to_full), _ptr(full_to_history),
                               _ptr(header), _ptr(score), _ptr(thres), _ptr(checkin_iter), int(glb_iter), M,
                               buffer_all.shape[0], hs, _ptr(ws), ws.numel(), _stream())
    _check(rc, "hc_record_history")


def get_graph_structure_score(ptr, idx, num_node, num_seed, num_layer):
    """Same signature as the reference (/root/reference/src/cpp/include/grad_check.h:22-24);
    level-synchronous and deterministic (the reference result depends on scheduling)."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    out = torch.empty(int(num_node), dtype=torch.int64, device=ptr.device)
    scratch = torch.empty(int(num_node), dtype=torch.int64, device=ptr.device)
    rc = lib.hc_structure_score(_ptr(ptr), _ptr(idx), ptr.numel() - 1, int(num_node), int(num_seed),
                                int(num_layer), _ptr(out), _ptr(scratch), _stream())
    _check(rc, "hc_structure_score")
    return out


def count_num(arr, mmax):
    """Histogram into int32[mmax+1] that skips value 0; same signature as the reference
    (/root/reference/src/cpp/include/grad_check.h:26)."""
    lib = load_library()
    _dev(arr, "arr", torch.int64)
    out = torch.empty(int(mmax) + 1, dtype=torch.int32, device=arr.device)
    rc = lib.hc_count_num(_ptr(arr), arr.numel(), int(mmax), _ptr(out), _stream())
    _check(rc, "hc_count_num")
    return out


# ----------------------------------------------------------------------------- extensions
def row_scores(grad, norm_kind=NORM_L2):
    """score[r] = ||grad[r]||_2 (or the L1 norm) in the library's fixed summation order."""
    lib = load_library()
    _dev(grad, "grad", torch.float32)
    if grad.dim() != 2:
        raise ValueError("grad must be [M, F]")
    M, F = grad.shape
    out = torch.empty(M, dtype=torch.float32, device=grad.device)
    _check(lib.hc_row_scores(_ptr(grad), _ptr(out), M, F, int(norm_kind), _stream()), "hc_row_scores")
    return out




def quantile_select(score, lo, hi, w, one_minus_w):
    """a + w*(b - a) (w < 0.5) or b - (b - a)*one_minus_w over the order statistics a, b of rank lo, hi of
    ``score`` (fp32 on the GPU), every step rounded to fp32, by a radix select instead of a sort: one launch
    by one block for the few thousand scores of a sampled batch, seven small launches over the whole chip for
    more than 32 768.  Returns a 1-element tensor."""
    lib = load_library()
    score = _dev(score, "score", torch.float32)
    n = score.numel()
    out = torch.empty(1, dtype=torch.float32, device=score.device)
    nbytes = int(lib.hc_quantile_workspace_bytes(n))      # 0 when one block takes them all
    ws = _workspace(nbytes, score.device)
    _check(lib.hc_quantile_threshold_ws(_ptr(score), n, int(lo), int(hi), float(w), float(one_minus_w), _ptr(out),
                                        _ptr(ws), ws.numel(), _stream()), "hc_quantile_threshold_ws")
    return out


def quantile_select_dev(score, n_dev, rate):
    """``quantile_threshold(score[:n], rate)`` with n read from ``n_dev`` (one int64 on the device, kept inside
    [1, len(score)]): the rank is worked out on the device as the host works it out, the same bits.  At most
    hc_quantile_max_scores() scores.  For recorded iterations."""
    lib = load_library()
    score = _dev(score, "score", torch.float32)
    _dev(n_dev, "n_dev", torch.int64)
    out = torch.empty(1, dtype=torch.float32, device=score.device)
    _check(lib.hc_quantile_threshold_dev(_ptr(score), _ptr(n_dev), score.numel(), float(rate), _ptr(out), _stream()),
           "hc_quantile_threshold_dev")
    return out


def stage_arrays(arrays, scalars_dst=None, scalars=()):
    """One launch that pads arrays into fixed-size ones and writes a few int64 scalars to device memory.
    ``arrays``: up to 16 tuples (src, dst, n_copy, fill) of contiguous device tensors, src of dst's dtype
    (elements of 8, 4, 2 or 1 bytes; they are moved as bit patterns): dst.view(-1)[i] = src.view(-1)[i] for
    i < n_copy, ``fill`` (an integer; 0 for floating-point data) behind.  ``scalars`` (up to 16 Python ints) go
    to ``scalars_dst[:len(scalars)]``."""
    lib = load_library()
    k = len(arrays)
    if k > 16 or len(scalars) > 16:
        raise ValueError("at most 16 arrays and 16 scalars per call")
    P, I64 = ctypes.c_void_p * max(k, 1), ctypes.c_int64 * max(k, 1)
    src, dst, n_copy, n_total, fill = P(), P(), I64(), I64(), I64()
    elem = (ctypes.c_int * max(k, 1))()
    for a, (s_, d_, n_, f_) in enumerate(arrays):
        _dev(d_, "dst")
        if d_.element_size() not in (8, 4, 2, 1) or not d_.is_contiguous():
            raise ValueError("staged arrays are contiguous tensors of 8-, 4-, 2- or 1-byte elements")
        n_ = int(n_)
        if n_ < 0 or n_ > d_.numel():
            raise ValueError("n_copy outside the destination")
        if n_ > 0:
            _dev(s_, "src", d_.dtype)
            if s_.numel() < n_ or not s_.is_contiguous():
                raise ValueError("source shorter than n_copy or not contiguous")
            src[a] = s_.data_ptr()
        dst[a], n_copy[a], n_total[a], fill[a] = d_.data_ptr(), n_, d_.numel(), int(f_)
        elem[a] = d_.element_size()
    vals = (ctypes.c_int64 * max(len(scalars), 1))(*[int(v) for v in scalars])
    if scalars:
        _dev(scalars_dst, "scalars_dst", torch.int64)
        if scalars_dst.numel() < len(scalars):
            raise ValueError("scalars_dst is too short")
    _check(lib.hc_stage_arrays(src, dst, n_copy, n_total, fill, elem, k, _ptr(scalars_dst) if scalars else _c_p(None),
                               vals, len(scalars), _stream()), "hc_stage_arrays")


def grad_check(grad, emb, slot, sub_to_full, thres, table, full2slot, slot2full, header, glb_iter,
               age=None, age_limit=0, used=None, checkin=None, norm_kind=NORM_L2, cmp_kind=CMP_LT,
               score=None, want_slots=False, static_scratch=False):
    """Fused admission pass (scores, predicate, mask, row-order ring slots, table scatter, maps).

    ``static_scratch=True`` goes through ``hc_grad_check_static``: the passes share a fixed device
    array inside the library instead of a workspace tensor (at most GRAD_CHECK_STATIC_MAX_ROWS rows;
    calls that overlap on one GPU race).

    ``grad`` [M,F] fp32 (or None with ``score`` given), ``emb`` [M,F] fp32, ``slot`` [M] int64
    (-1 = not cached), ``thres`` 1-element fp32 device tensor, ``table`` [capacity,F]
    fp32/fp16/bf16, maps int64, ``header`` 1-element int64 device tensor (advanced in place).
    Returns (mask[bool], score[f32]) and the per-row slot when ``want_slots``."""
    lib = load_library()
    _dev(emb, "emb", torch.float32)
    M, F = emb.shape
    dev = emb.device
    if grad is not None:
        _dev(grad, "grad", torch.float32)
        if tuple(grad.shape) != (M, F):
            raise ValueError("grad and emb must have the same shape")
    elif score is None:
        raise ValueError("either grad or score is required")
    else:
        _dev(score, "score", torch.float32)
    _dev(slot, "slot", torch.int64)
    _dev(sub_to_full, "sub_to_full", torch.int64)
    thres = _dev(thres.reshape(1), "thres", torch.float32)
    _dev(table, "table")
    if table.dim() != 2 or table.shape[1] != F:
        raise ValueError("table must be [capacity, F]")
    for t, n in ((full2slot, "full2slot"), (slot2full, "slot2full"), (header, "header")):
        _dev(t, n, torch.int64)
    if slot2full.numel() < table.shape[0]:
        raise ValueError("slot2full is shorter than the table")
    if age is not None:
        _dev(age, "age", torch.int32)
    if used is not None:
        _dev(used, "used")
        if used.dtype not in (torch.bool, torch.uint8):
            raise ValueError("used must be bool")
    if checkin is not None:
        _dev(checkin, "checkin", torch.int64)
    # every per-row argument must cover the M rows of emb: the kernels trust their lengths
    for t, n in ((slot, "slot"), (sub_to_full, "sub_to_full"), (age, "age"), (used, "used"), (score, "score")):
        if t is not None and t.numel() < M:
            raise ValueError(f"{n} has {t.numel()} entries, emb has {M} rows")
    mask = torch.empty(M, dtype=torch.uint8, device=dev)
    score_out = torch.empty(M, dtype=torch.float32, device=dev)
    slot_out = torch.empty(M, dtype=torch.int64, device=dev) if want_slots else None
    iter_on_device = isinstance(glb_iter, torch.Tensor)       # recorded iterations: one int64 on the device
    if iter_on_device:
        _dev(glb_iter, "glb_iter", torch.int64)
        if static_scratch:
            raise ValueError("glb_iter on the device goes with a workspace")
    args = (_ptr(grad), _ptr(score), _ptr(emb), _ptr(slot), _ptr(age), _ptr(used),
            _ptr(sub_to_full), _ptr(thres), int(age_limit), int(norm_kind), int(cmp_kind),
            _ptr(mask), _ptr(score_out), _ptr(slot_out), _ptr(table),
            _float_dtype(table, "table"), table.shape[0], _ptr(full2slot), _ptr(slot2full),
            _ptr(checkin), _ptr(header), _ptr(glb_iter) if iter_on_device else int(glb_iter), M, F)
    if iter_on_device:
        ws = _workspace(lib.hc_grad_check_workspace_bytes(M), dev)
        _check(lib.hc_grad_check_dev(*args, _ptr(ws), ws.numel(), _stream()), "hc_grad_check_dev")
    elif static_scratch:
        with torch.cuda.device(dev):
            _check(lib.hc_grad_check_static(*args, _stream()), "hc_grad_check_static")
    else:
        ws = _workspace(lib.hc_grad_check_workspace_bytes(M), dev)
        _check(lib.hc_grad_check(*args, _ptr(ws), ws.numel(), _stream()), "hc_grad_check")
    if want_slots:
        return mask.view(torch.bool), score_out, slot_out
    return mask.view(torch.bool), score_out


def cache_append(score, thres, emb, sub2embed, sub_to_full, buffer, hidden, in_channels, full2embed,
                 embed2full, feat2full, header, overflow=None):
    """Append-only admission of HistoryCache.update_history
    (/root/reference/hiscache/history_cache.py:215-254) as one launch sequence.
    ``buffer`` is the flat fp32 cache; ``header`` / ``overflow`` are 1-element int64 device tensors.
    Returns the admission mask."""
    lib = load_library()
    _dev(score, "score", torch.float32)
    _dev(emb, "emb", torch.float32)
    M = emb.shape[0]
    H = int(hidden)
    if emb.dim() != 2 or emb.shape[1] != H:
        raise ValueError("emb must be [M, hidden]")
    thres = _dev(thres.reshape(1), "thres", torch.float32)
    _dev(buffer, "buffer", torch.float32)
    capacity = buffer.numel() // H
    for t, n in ((sub2embed, "sub2embed"), (sub_to_full, "sub_to_full"), (full2embed, "full2embed"),
                 (embed2full, "embed2full"), (header, "header")):
        _dev(t, n, torch.int64)
    for t, n in ((score, "score"), (sub2embed, "sub2embed"), (sub_to_full, "sub_to_full")):
        if t.numel() < M:
            raise ValueError(f"{n} has {t.numel()} entries, emb has {M} rows")
    if embed2full.numel() < capacity:
        capacity = embed2full.numel()
    n_feat = 0
    if feat2full is not None and feat2full.numel() > 0:
        _dev(feat2full, "feat2full", torch.int64)
        n_feat = feat2full.numel()
    else:
        feat2full = None
    if overflow is not None:
        _dev(overflow, "overflow", torch.int64)
    mask = torch.empty(M, dtype=torch.uint8, device=emb.device)
    ws = _workspace(lib.hc_grad_check_workspace_bytes(M), emb.device)
    rc = lib.hc_cache_append(_ptr(score), _ptr(thres), _ptr(emb), _ptr(sub2embed), _ptr(sub_to_full),
                             _ptr(mask), _ptr(buffer), capacity, H, int(in_channels), _ptr(full2embed),
                             _ptr(embed2full), _ptr(feat2full), n_feat, _ptr(header), _ptr(overflow), M,
                             _ptr(ws), ws.numel(), _stream())
    _check(rc, "hc_cache_append")
    return mask.view(torch.bool)


def gather_rows(src, ids, mask=None, out=None, accumulate=False, out_dtype=torch.float32, stream=None):
    """out[i] = src[ids[i]] where mask[i] (else 0), as ``out_dtype`` (fp32 by default).  ``src`` may be
    a GPU tensor or a pinned host tensor (read zero-copy over the host link).  Negative ids index
    from the end.  ``stream`` (a torch stream; default: the current one): where the kernel is enqueued --
    a new ``out`` still comes from the current stream's memory, so a caller that names another stream
    records it on ``out`` (``out.record_stream(stream)``) and orders the two streams itself."""
    lib = load_library()
    if not isinstance(src, torch.Tensor) or src.dim() != 2 or not src.is_contiguous():
        raise ValueError("src must be a contiguous 2-D tensor")
    if not src.is_cuda and not src.is_pinned():
        raise RuntimeError("src must be on the GPU or in pinned host memory")
    _dev(ids, "ids", torch.int64)
    n, F = ids.numel(), src.shape[1]
    if mask is not None:
        _dev(mask, "mask")
        if mask.dtype not in (torch.bool, torch.uint8) or mask.numel() < n:
            raise ValueError("mask must be a bool tensor with one entry per id")
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an existing out tensor")
        out = torch.empty((n, F), dtype=out_dtype, device=ids.device)
    else:
        _dev(out, "out")
        if tuple(out.shape) != (n, F):
            raise ValueError("out must be [len(ids), F]")
    rc = lib.hc_gather_rows(_ptr(src), _float_dtype(src, "src"), src.shape[0], _ptr(ids), _ptr(mask),
                            _ptr(out), _float_dtype(out, "out"), 1 if accumulate else 0, n, F,
                            _stream() if stream is None else _c_p(stream.cuda_stream))
    _check(rc, "hc_gather_rows")
    return out


def gather_rows_hot(hot, slot_map, ids, mask=None, out=None, out_dtype=torch.float32, cold=None, stream=None):
    """The device-memory tier of a two-tier feature matrix: ``hot`` [n_hot, F] holds copies of the most
    requested rows, ``slot_map`` (int32, one entry per node) a node's row in it or -1.  out[i] = hot row of
    ids[i] where mask[i] and the node has one, 0 where not mask[i]; the other rows are left alone and flagged in
    ``cold`` (uint8, one per id) for ``gather_rows_flagged``.  Returns (out, cold)."""
    lib = load_library()
    _dev(hot, "hot")
    if hot.dim() != 2 or not hot.is_contiguous():
        raise ValueError("hot must be a contiguous [n_hot, F] tensor")
    _dev(slot_map, "slot_map", torch.int32)
    _dev(ids, "ids", torch.int64)
    n, F = ids.numel(), hot.shape[1]
    if mask is not None:
        _dev(mask, "mask")
        if mask.dtype not in (torch.bool, torch.uint8) or mask.numel() < n:
            raise ValueError("mask must be a bool tensor with one entry per id")
    if out is None:
        out = torch.empty((n, F), dtype=out_dtype, device=ids.device)
    else:
        _dev(out, "out")
        if tuple(out.shape) != (n, F):
            raise ValueError("out must be [len(ids), F]")
    if cold is None:
        cold = torch.empty(n, dtype=torch.uint8, device=ids.device)
    else:
        _dev(cold, "cold", torch.uint8)
        if cold.numel() < n:
            raise ValueError("cold must hold one byte per id")
    rc = lib.hc_gather_rows_hot(_ptr(hot), _float_dtype(hot, "hot"), hot.shape[0], _ptr(slot_map), slot_map.numel(),
                                _ptr(ids), _ptr(mask), _ptr(out), _float_dtype(out, "out"), _ptr(cold), n, F,
                                _stream() if stream is None else _c_p(stream.cuda_stream))
    _check(rc, "hc_gather_rows_hot")
    return out, cold


def gather_rows_flagged(src, ids, flag, out, stream=None):
    """out[i] = src[ids[i]] for the rows with flag[i] (uint8), every other row of ``out`` is left as it is.
    ``src`` may be a GPU tensor or a pinned host tensor (read zero-copy over the host link)."""
    lib = load_library()
    if not isinstance(src, torch.Tensor) or src.dim() != 2 or not src.is_contiguous():
        raise ValueError("src must be a contiguous 2-D tensor")
    if not src.is_cuda and not src.is_pinned():
        raise RuntimeError("src must be on the GPU or in pinned host memory")
    _dev(ids, "ids", torch.int64)
    _dev(flag, "flag")
    _dev(out, "out")
    n, F = ids.numel(), src.shape[1]
    if flag.dtype not in (torch.bool, torch.uint8) or flag.numel() < n:
        raise ValueError("flag must hold one byte per id")
    if tuple(out.shape) != (n, F):
        raise ValueError("out must be [len(ids), F]")
    rc = lib.hc_gather_rows_flagged(_ptr(src), _float_dtype(src, "src"), src.shape[0], _ptr(ids), _ptr(flag),
                                    _ptr(out), _float_dtype(out, "out"), n, F,
                                    _stream() if stream is None else _c_p(stream.cuda_stream))
    _check(rc, "hc_gather_rows_flagged")
    return out


_cu_stream_handles = []


def _destroy_cu_streams():
    """At interpreter exit: wait for the device and give the CU-limited streams back while the HIP runtime is
    still up (a stream of this kind left to the runtime's own teardown crashed a profiled run at exit: a
    host-side crash in the process's teardown, after all results were out; no kernel was running).  Safe to
    call any number of times: a handle is destroyed once."""
    if not _cu_stream_handles:
        return
    try:
        torch.cuda.synchronize()
    except Exception:
        pass
    lib = load_library()
    while _cu_stream_handles:
        handle = _cu_stream_handles.pop()
        _forget_stream(handle)
        lib.hc_stream_destroy(_c_p(handle))


def _forget_stream(handle):
    """Drop what this module keeps per stream (scratch buffer, epilogue ticket) for a stream that goes away."""
    for table in (_ws_cache, _tickets):
        for key in [k for k in table if k[1] == handle]:
            del table[key]


def streams_share_queue(a, b, device=None, chain=16):
    """Do the torch streams ``a`` and ``b`` share a hardware queue?  Found by measurement: a chain of fills is queued
    on ``b``, then one small launch on ``a``; on a queue of its own that launch is done long before the chain is.
    The runtime hands its streams a few hardware queues (four by default) in the order of their first use, so two
    streams that a program means to run side by side may turn out to take turns, and there is no call that tells."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if a.cuda_stream == b.cuda_stream:
        return True
    # 256 MB: about 60 us per fill, a millisecond in all -- several times what the host needs to queue the chain,
    # a tracer's overhead included (were the chain over before the small launch is queued, the answer would be "yes")
    big = torch.empty(1 << 26, device=device)
    small = torch.zeros(256, device=device)
    torch.cuda.synchronize(device)
    b0, b1, a1 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    with torch.cuda.stream(b):
        b0.record()
        for _ in range(int(chain)):
            big.fill_(1.0)
        b1.record()
    with torch.cuda.stream(a):
        small.add_(1.0)
        a1.record()
    torch.cuda.synchronize(device)
    return b0.elapsed_time(a1) >= 0.9 * b0.elapsed_time(b1)


def stream_apart_from(others, device=None, candidates=8):
    """A torch stream (default priority) that shares its hardware queue with none of ``others`` (see
    ``streams_share_queue``): up to ``candidates`` new streams are tried, the last one is returned if none passes.
    For the few long-lived streams of a training loop (the sampler's, the iteration's), made once."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    cand = None
    for _ in range(max(1, int(candidates))):
        cand = torch.cuda.Stream(device=device)
        if not any(streams_share_queue(cand, o, device) for o in others):
            break
    return cand


def release_cu_limited_stream(stream):
    """Give a stream made by ``cu_limited_stream`` back before the interpreter exits: waits for its work,
    destroys it and drops the scratch this module kept for it.  The torch wrapper must not be used afterwards.
    Unknown or already released streams are ignored."""
    handle = int(stream.cuda_stream)
    if handle not in _cu_stream_handles:
        return False
    stream.synchronize()
    _cu_stream_handles.remove(handle)
    _forget_stream(handle)
    load_library().hc_stream_destroy(_c_p(handle))
    return True


def cu_limited_stream(n_cus, device):
    """A torch stream (default priority) whose kernels run on ``n_cus`` compute units only, spread over the
    chip: for work that waits on the host link beside compute (``PinnedFeatureStore.prefetch``).  The
    stream lives until the interpreter exits.  (The runtime has refused masks of 2 and of 4 units on an MI355X;
    8 -- one per die -- and more work.)"""
    lib = load_library()
    device = torch.device(device)
    handle = ctypes.c_void_p()
    with torch.cuda.device(device):
        rc = lib.hc_stream_create_cu_limited(int(n_cus), ctypes.cast(ctypes.pointer(handle), _c_p))
        if rc == 3:                                  # HC_ELAUNCH: the runtime said no
            raise RuntimeError(f"the runtime refused a stream kept to {int(n_cus)} compute units (masks of fewer than 8 "
                               "units, one per die, have been refused on this GPU)")
        _check(rc, "hc_stream_create_cu_limited")
    if not _cu_stream_handles:
        import atexit
        atexit.register(_destroy_cu_streams)
    _cu_stream_handles.append(handle.value)
    return torch.cuda.ExternalStream(handle.value, device=device)


STAT_NAMES = ("lookups", "nodes", "one_hop_nodes", "embedding_hits", "nodes_pruned", "feature_hits", "rows_loaded",
              "rows_admitted")


def load_mask(used, sub2feat=None, sub2embed=None, prev_mask=None, counters=None, want_masks=True):
    """(hit_feat_mask, load_mask) of a batch -- ``load = used & ~(sub2feat != -1)``, the rows that have to come
    from the feature store (/root/reference/hiscache/history_cache.py:327-330) -- in one launch that also adds the
    batch's hit counts (and the rows admitted by ``prev_mask``) to ``counters`` (int64[8] on the device, order
    ``STAT_NAMES``).  Without a feature cache (``sub2feat`` None) the load mask is ``used`` itself and only the
    counters are touched: (None, used) is returned."""
    lib = load_library()
    _dev(used, "used")
    if used.element_size() != 1:
        raise ValueError("used must hold one byte per node")
    n_all = used.numel()
    n1 = 0 if sub2embed is None else _dev(sub2embed, "sub2embed", torch.int64).numel()
    n_prev = 0
    if prev_mask is not None:
        _dev(prev_mask, "prev_mask")
        if prev_mask.element_size() != 1:
            raise ValueError("prev_mask must hold one byte per row")
        n_prev = prev_mask.numel()
    hit = load = None
    if sub2feat is not None:
        _dev(sub2feat, "sub2feat", torch.int64)
        if sub2feat.numel() < n_all:
            raise ValueError("sub2feat is shorter than used")
        if want_masks:
            hit = torch.empty(n_all, dtype=torch.bool, device=used.device)
            load = torch.empty(n_all, dtype=torch.bool, device=used.device)
    if counters is not None:
        _dev(counters, "counters", torch.int64)
        if counters.numel() < len(STAT_NAMES):
            raise ValueError("counters must hold %d entries" % len(STAT_NAMES))
    rc = lib.hc_load_mask(_ptr(used), _ptr(sub2feat), _ptr(sub2embed), _ptr(prev_mask), n_all, n1, n_prev,
                          _ptr(hit), _ptr(load), _ptr(counters), _stream())
    _check(rc, "hc_load_mask")
    return hit, (load if sub2feat is not None else used)


def fixup_rows(src, ids, need, have, out):
    """``out`` holds ``gather_rows(src, ids, mask=have)`` (rows read ahead of time under a guess); bring it
    to ``gather_rows(src, ids, mask=need)`` in place: rows that are needed but were not read are read,
    rows that were read but are not needed are cleared, the others are not touched."""
    lib = load_library()
    if not isinstance(src, torch.Tensor) or src.dim() != 2 or not src.is_contiguous():
        raise ValueError("src must be a contiguous 2-D tensor")
    if not src.is_cuda and not src.is_pinned():
        raise RuntimeError("src must be on the GPU or in pinned host memory")
    _dev(ids, "ids", torch.int64)
    _dev(out, "out")
    n, F = ids.numel(), src.shape[1]
    if tuple(out.shape) != (n, F):
        raise ValueError("out must be [len(ids), F]")
    for name, m in (("need", need), ("have", have)):
        _dev(m, name)
        if m.dtype not in (torch.bool, torch.uint8) or m.numel() < n:
            raise ValueError(f"{name} must be a bool tensor with one entry per id")
    rc = lib.hc_fixup_rows(_ptr(src), _float_dtype(src, "src"), src.shape[0], _ptr(ids), _ptr(need), _ptr(have),
                           _ptr(out), _float_dtype(out, "out"), n, F, _stream())
    _check(rc, "hc_fixup_rows")
    return out


def lookup(map_tensor, ids, offset=0, n_valid=None):
    """out[i] = map[ids[i] + offset] (int64 gather; negative positions index from the end).  ``n_valid`` (a
    one-element int64 device tensor, for recorded iterations): entries at or behind it are padding and give -1."""
    lib = load_library()
    _dev(map_tensor, "map", torch.int64)
    _dev(ids, "ids", torch.int64)
    out = torch.empty(ids.numel(), dtype=torch.int64, device=ids.device)
    if n_valid is not None:
        _dev(n_valid, "n_valid", torch.int64)
        rc = lib.hc_lookup_dev(_ptr(map_tensor), map_tensor.numel(), _ptr(ids), int(offset), _ptr(n_valid), _ptr(out),
                               ids.numel(), _stream())
        _check(rc, "hc_lookup_dev")
        return out
    rc = lib.hc_lookup(_ptr(map_tensor), map_tensor.numel(), _ptr(ids), int(offset), _ptr(out), ids.numel(),
                       _stream())
    _check(rc, "hc_lookup")
    return out


def ring_lookup(full2slot, ids, table, checkin=None, now=0, age_limit=1 << 62, want_rows=True, n_valid=None):
    """Slots of ``ids`` in a ring table and the table rows of the hits, in one launch.  An entry with
    ``now - checkin[slot] >= age_limit`` counts as absent (-1).  Returns (slot[int64], rows[fp32] or
    None); rows of absent ids are zero.  For recorded iterations ``now`` may be a one-element int64 device
    tensor, together with ``n_valid`` (the same): ids behind the first ``n_valid`` are padding and find nothing."""
    lib = load_library()
    _dev(full2slot, "full2slot", torch.int64)
    _dev(ids, "ids", torch.int64)
    _dev(table, "table")
    if table.dim() != 2:
        raise ValueError("table must be [capacity, F]")
    if checkin is not None:
        _dev(checkin, "checkin", torch.int64)
        if checkin.numel() < table.shape[0]:
            raise ValueError("checkin is shorter than the table")
    n = ids.numel()
    slot = torch.empty(n, dtype=torch.int64, device=ids.device)
    rows = torch.empty((n, table.shape[1]), dtype=torch.float32, device=ids.device) if want_rows else None
    if isinstance(now, torch.Tensor) or n_valid is not None:
        if not isinstance(now, torch.Tensor) or n_valid is None:
            raise ValueError("now and n_valid go together as one-element int64 device tensors")
        _dev(now, "now", torch.int64)
        _dev(n_valid, "n_valid", torch.int64)
        rc = lib.hc_ring_lookup_dev(_ptr(full2slot), full2slot.numel(), _ptr(ids), _ptr(checkin), _ptr(now),
                                    _ptr(n_valid), int(age_limit), _ptr(table), _float_dtype(table, "table"),
                                    table.shape[0], table.shape[1], _ptr(slot), _ptr(rows), n, _stream())
        _check(rc, "hc_ring_lookup_dev")
        return slot, rows
    rc = lib.hc_ring_lookup(_ptr(full2slot), full2slot.numel(), _ptr(ids), _ptr(checkin), int(now), int(age_limit),
                            _ptr(table), _float_dtype(table, "table"), table.shape[0], table.shape[1], _ptr(slot),
                            _ptr(rows), n, _stream())
    _check(rc, "hc_ring_lookup")
    return slot, rows


MAX_TYPED_RELATIONS = 64


def typed_csr(ptr, idx, edge_types, num_rel, num_node, n_src, used_mask=None, want_weights=False):
    """Regroup the edges of the first ``num_node`` rows by (row, relation), keeping the edge order
    inside every group.  Returns (ptr2[num_node*num_rel+1], idx2, cnt[num_node, num_rel], deg[num_node]);
    edges with a relation outside [0, num_rel), a source outside [0, n_src) or a source that
    ``used_mask`` (bool[n_src]) rules out are dropped.  Only the first ptr2[-1] entries of idx2 are
    defined.  The grouping the reference obtains from a per-call sort by relation
    (/root/reference/hiscache/history_model.py:248-270).  With ``want_weights`` a fifth result holds,
    beside every entry of idx2, 1/deg of its row (fp32): the edge values that turn the weighted
    aggregation over the groups into each group's share of the row's mean."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    _dev(edge_types, "edge_types", torch.int64)
    R, K = int(num_node), int(num_rel)
    if K < 1 or K > MAX_TYPED_RELATIONS:
        raise ValueError("num_rel must be in [1, %d]" % MAX_TYPED_RELATIONS)
    if ptr.numel() < R + 1:
        raise ValueError("ptr is shorter than num_node + 1")
    E = min(int(edge_types.numel()), int(idx.numel()))
    if used_mask is not None:
        _dev(used_mask, "used_mask")
        if used_mask.dtype not in (torch.bool, torch.uint8):
            raise ValueError("used_mask must be bool or uint8")
        if used_mask.numel() < int(n_src):
            raise ValueError("used_mask is shorter than n_src")
    dev = ptr.device
    ptr2 = torch.empty(R * K + 1, dtype=torch.int64, device=dev)
    idx2 = torch.empty(max(E, 1), dtype=torch.int64, device=dev)
    cnt = torch.empty(R * K, dtype=torch.int64, device=dev)
    deg = torch.empty(R, dtype=torch.int64, device=dev)
    weights = torch.empty(max(E, 1), dtype=torch.float32, device=dev) if want_weights else None
    if R * K <= TYPED_CSR_SMALL_GROUPS:
        # sampled batches: the count kernel's last block scans the group sizes (no workspace, no library call)
        rc = lib.hc_typed_csr(_ptr(ptr), _ptr(idx), _ptr(edge_types), _ptr(used_mask), R, E, int(n_src), K,
                              _ptr(ptr2), _ptr(idx2), _ptr(cnt), _ptr(deg), _ptr(weights), _c_p(None), 0,
                              _ptr(_ticket(dev)), _stream())
    else:
        ws_bytes = int(lib.hc_typed_csr_workspace_bytes(R, K))
        ws = _workspace(ws_bytes, dev)
        rc = lib.hc_typed_csr(_ptr(ptr), _ptr(idx), _ptr(edge_types), _ptr(used_mask), R, E, int(n_src), K,
                              _ptr(ptr2), _ptr(idx2), _ptr(cnt), _ptr(deg), _ptr(weights), _ptr(ws), ws_bytes,
                              _c_p(None), _stream())
    _check(rc, "hc_typed_csr")
    if want_weights:
        return ptr2, idx2, cnt.view(R, K), deg, weights
    return ptr2, idx2, cnt.view(R, K), deg


def edge_types_by_ranges(ptr, idx, sub_to_full, num_node, bounds, pair_to_rel):
    """out[e] = pair_to_rel[type(row of e), type(idx[e])] for the edges of the first ``num_node`` rows,
    where a node's type is the number of entries of ``bounds`` (ascending int64 tensor) its full id
    has reached; other entries of the result are -1."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    _dev(sub_to_full, "sub_to_full", torch.int64)
    _dev(bounds, "bounds", torch.int64)
    _dev(pair_to_rel, "pair_to_rel", torch.int64)
    T = bounds.numel() + 1
    if pair_to_rel.numel() != T * T:
        raise ValueError("pair_to_rel must be [T, T] with T = len(bounds) + 1")
    R = int(num_node)
    if ptr.numel() < R + 1:
        raise ValueError("ptr is shorter than num_node + 1")
    out = torch.empty(idx.numel(), dtype=torch.int64, device=idx.device)      # the call writes every entry
    rc = lib.hc_edge_types_by_ranges(_ptr(ptr), _ptr(idx), _ptr(sub_to_full), sub_to_full.numel(), _ptr(bounds),
                                     int(bounds.numel()), _ptr(pair_to_rel), _ptr(out), R, idx.numel(), _stream())
    _check(rc, "hc_edge_types_by_ranges")
    return out


# ------------------------------------------------------------------ layer epilogue
BN_RELU_MAX_CHANNELS = 1024
TYPED_CSR_SMALL_GROUPS = 1 << 20
_tickets = {}


def _ticket(device):
    """The zeroed word the epilogue kernels count their blocks in (one per device and stream; the
    kernels leave it zero)."""
    key = (device.index, _raw_stream(device.index))
    t = _tickets.get(key)
    if t is None:
        t = _tickets[key] = torch.zeros(64, dtype=torch.int32, device=device)
    return t


def prepare_stream(device):
    """Create what this module keeps per stream (the epilogue kernels' ticket word) for torch's current stream
    now, so that a recording on that stream allocates and clears nothing of the kind."""
    _ticket(torch.device(device))


def bn_relu_supported(x, channels):
    return x.is_cuda and x.dtype == torch.float32 and channels % 4 == 0 and 4 <= channels <= BN_RELU_MAX_CHANNELS


class _BiasBnRelu(torch.autograd.Function):
    """relu(batch_norm(x + bias)) in training mode as one autograd node over ``hc_bn_relu_fwd`` /
    ``hc_bn_relu_bwd`` (/root/reference/hiscache/history_model.py:139-140).  ``x`` comes WITHOUT the
    bias; the running statistics are updated in place."""

    @staticmethod
    def forward(ctx, x, bias, gamma, beta, running_mean, running_var, momentum, eps, batches_tracked=None,
                n_dev=None):
        lib = load_library()
        n, C = x.shape
        y = torch.empty_like(x)
        stats = torch.empty((2, C), dtype=torch.float32, device=x.device)      # mean, 1/sqrt(var + eps)
        ws = _workspace(lib.hc_bn_relu_workspace_bytes(n, C), x.device)
        sp = stats.data_ptr()
        _check(lib.hc_bn_relu_fwd_dev(_ptr(x), _ptr(bias), _ptr(gamma), _ptr(beta), _ptr(running_mean),
                                      _ptr(running_var), _ptr(batches_tracked), float(momentum), float(eps), _ptr(y),
                                      _c_p(sp), _c_p(sp + 4 * C), n, C, _ptr(n_dev), _ptr(ws), ws.numel(),
                                      _ptr(_ticket(x.device)), _stream()), "hc_bn_relu_fwd")
        ctx.save_for_backward(x, stats, gamma if gamma is not None else x.new_empty(0),
                              beta if beta is not None else x.new_empty(0))
        ctx.hc = (bias is not None, gamma is not None, beta is not None, n_dev)
        return y

    @staticmethod
    def backward(ctx, dy):
        lib = load_library()
        x, stats, gamma, beta = ctx.saved_tensors
        has_bias, has_gamma, has_beta, n_dev = ctx.hc
        dy = dy.contiguous()
        n, C = x.shape
        dx = torch.empty_like(x)
        grads = torch.empty((3, C), dtype=torch.float32, device=x.device)     # dgamma, dbeta, dbias
        ws = _workspace(lib.hc_bn_relu_workspace_bytes(n, C), x.device)
        sp, gp = stats.data_ptr(), grads.data_ptr()
        _check(lib.hc_bn_relu_bwd_dev(_ptr(dy), _ptr(x), _ptr(gamma if has_gamma else None),
                                      _ptr(beta if has_beta else None), _c_p(sp), _c_p(sp + 4 * C), _ptr(dx),
                                      _c_p(gp), _c_p(gp + 4 * C), _c_p(gp + 8 * C if has_bias else None), n, C,
                                      _ptr(n_dev), _ptr(ws), ws.numel(), _ptr(_ticket(x.device)), _stream()),
               "hc_bn_relu_bwd")
        return (dx, grads[2] if has_bias else None, grads[0] if has_gamma else None,
                grads[1] if has_beta else None, None, None, None, None, None, None)


def weight_grad_supported(g, x):
    return (g.is_cuda and g.dtype == torch.float32 and x.dtype == torch.float32 and g.dim() == 2 and x.dim() == 2
            and g.shape[1] % 64 == 0 and x.shape[1] % 64 == 0 and g.shape[1] <= 4096 and x.shape[1] <= 4096
            and g.shape[0] >= 1)


def weight_grad(g, x0, x1=None):
    """``g.t() @ x0`` (and ``g.t() @ x1``): the weight gradients of a layer's linear maps on the matrix
    cores, rows split into slabs that are added in a fixed order.  g [n, H], x [n, F], fp32."""
    lib = load_library()
    _dev(g, "g", torch.float32)
    _dev(x0, "x0", torch.float32)
    if x1 is not None:
        _dev(x1, "x1", torch.float32)
        if x1.shape != x0.shape:
            raise ValueError("x1 must have x0's shape")
    if g.dim() != 2 or x0.dim() != 2 or x0.shape[0] != g.shape[0]:
        raise ValueError("g [n, H] and x [n, F] must have the same number of rows")
    n, H = g.shape
    F = x0.shape[1]
    n_op = 1 if x1 is None else 2
    dw = torch.empty((n_op, H, F), dtype=torch.float32, device=g.device)
    ws = _workspace(lib.hc_weight_grad_workspace_bytes(n, H, F, n_op), g.device)
    p = dw.data_ptr()
    _check(lib.hc_weight_grad(_ptr(g), _ptr(x0), _ptr(x1), n, H, F, _c_p(p),
                              _c_p(p + 4 * H * F) if x1 is not None else _c_p(None), _ptr(ws), ws.numel(),
                              _stream()), "hc_weight_grad")
    return (dw[0], dw[1]) if x1 is not None else dw[0]


def bias_bn_relu(x, bias, gamma, beta, running_mean, running_var, momentum, eps, num_batches_tracked=None,
                 n_dev=None):
    """Training-mode ``relu(batch_norm(x + bias))``; x is [n, C] fp32 on the GPU, n >= 2.
    ``num_batches_tracked`` (one int64 on the device, optional) is incremented by the call's first kernel.
    ``n_dev`` (one int64 on the device, optional; for recorded iterations): only the first ``n_dev`` rows are in
    use; the others stay out of the statistics, get zeros in the output and a zero gradient."""
    _dev(x, "x")
    if x.dim() != 2:
        raise ValueError("x must be [n, C]")
    if x.shape[0] < 2:
        raise ValueError("Expected more than 1 value per channel when training, got input size %s"
                         % (tuple(x.shape),))
    if not bn_relu_supported(x, x.shape[1]):
        raise ValueError("hc_bn_relu: fp32 on the GPU with C % 4 == 0 and C <= 1024")
    for name, t in (("bias", bias), ("gamma", gamma), ("beta", beta), ("running_mean", running_mean),
                    ("running_var", running_var)):
        if t is not None:
            _dev(t, name, torch.float32)
            if t.numel() != x.shape[1]:
                raise ValueError(f"{name} must hold C = {x.shape[1]} values")
    if num_batches_tracked is not None:
        _dev(num_batches_tracked, "num_batches_tracked", torch.int64)
        if num_batches_tracked.numel() != 1:
            raise ValueError("num_batches_tracked must hold one value")
    if n_dev is not None:
        _dev(n_dev, "n_dev", torch.int64)
    return _BiasBnRelu.apply(x, bias, gamma, beta, running_mean, running_var, momentum, eps, num_batches_tracked,
                             n_dev)


def evict(checkin, slot2full, full2slot, stale_iter, sub2slot=None, score=None, thres=None):
    """Give up table slots in place: every slot with -1 < checkin <= ``stale_iter`` and, when
    ``sub2slot`` / ``score`` / ``thres`` (1-element fp32 device tensor) are given, the slot of every
    batch row whose score is >= thres (/root/reference/hiscache/history_table.py:189-251)."""
    lib = load_library()
    _dev(checkin, "checkin", torch.int64)
    _dev(slot2full, "slot2full", torch.int64)
    _dev(full2slot, "full2slot", torch.int64)
    M = 0
    if sub2slot is not None:
        _dev(sub2slot, "sub2slot", torch.int64)
        _dev(score, "score", torch.float32)
        _dev(thres, "thres", torch.float32)
        M = sub2slot.numel()
        if score.numel() < M:
            raise ValueError("score is shorter than sub2slot")
    cap = slot2full.numel()
    if checkin.numel() < cap:
        raise ValueError("checkin is shorter than slot2full")
    rc = lib.hc_evict(_ptr(sub2slot), _ptr(score), _ptr(thres), M, int(stale_iter), _ptr(checkin), _ptr(slot2full),
                      _ptr(full2slot), cap, full2slot.numel(), _stream())
    _check(rc, "hc_evict")


def sample_map(num_nodes, device):
    """The sampler's persistent node map (int32[num_nodes], every entry "unseen")."""
    lib = load_library()
    m = torch.empty(int(num_nodes), dtype=torch.int32, device=device)
    with torch.cuda.device(m.device):
        _check(lib.hc_sample_map_init(_ptr(m), m.numel(), _stream()), "hc_sample_map_init")
    return m


def sample_capacity(n_seed, fanout, num_nodes):
    """(max_rows, max_edges, max_nodes) a batch of ``n_seed`` seeds can reach."""
    lib = load_library()
    fan = (ctypes.c_int64 * len(fanout))(*[int(f) for f in fanout])
    out = [ctypes.c_int64(0) for _ in range(3)]
    rc = lib.hc_sample_capacity(int(n_seed), ctypes.cast(fan, _c_p), len(fanout), int(num_nodes),
                                *[ctypes.cast(ctypes.pointer(o), _c_p) for o in out])
    _check(rc, "hc_sample_capacity")
    return tuple(int(o.value) for o in out)


def build_transpose_dev(ptr, idx, rows_dev, edges_dev, nodes_dev, max_edges, max_nodes, want_edges=False,
                        overflow=None, max_in_degree=None):
    """The transposed view of a block whose sizes are still on the device (one-element int64 views
    ``rows_dev``, ``edges_dev``, ``nodes_dev``, e.g. slices of the sampler's ``counts``): returns
    (ptrT, rowT, edgeT) at the capacities ``max_nodes + 1`` / ``max_edges``; nothing is read back.
    ``overflow`` (one int32 on the device, optional) is set to 1 when a size exceeded its capacity and the
    view is that of the truncated block, else to 0.  ``max_in_degree`` (a one-element int64 view on the device,
    optional) receives the largest number of edges one source has in the view."""
    lib = load_library()
    _dev(ptr, "ptr", torch.int64)
    _dev(idx, "idx", torch.int64)
    if max_in_degree is not None and _dev(max_in_degree, "max_in_degree", torch.int64).numel() < 1:
        raise ValueError("max_in_degree is empty")
    for t, name in ((rows_dev, "rows_dev"), (edges_dev, "edges_dev"), (nodes_dev, "nodes_dev")):
        _dev(t, name, torch.int64)
        if t.numel() < 1:
            raise ValueError(f"{name} is empty")
    max_edges, max_nodes = int(max_edges), int(max_nodes)
    if idx.numel() < max_edges:
        raise ValueError("idx is shorter than max_edges")
    dev = ptr.device
    nbytes = int(lib.hc_transpose_dev_workspace_bytes(max_edges, max_nodes))
    if nbytes == 0:
        raise ValueError("block too large for the device-sized transposed view (2^24 edges / nodes)")
    ptrT = torch.empty(max_nodes + 1, dtype=torch.int64, device=dev)
    rowT = torch.empty(max(max_edges, 1), dtype=torch.int32, device=dev)
    edgeT = torch.empty(max(max_edges, 1), dtype=torch.int32, device=dev) if want_edges else None
    ws = _workspace(nbytes, dev)
    rc = lib.hc_build_transpose_dev_deg(_ptr(ptr), _ptr(idx), _ptr(rows_dev), _ptr(edges_dev), _ptr(nodes_dev),
                                        max_edges, max_nodes, _ptr(ptrT), _ptr(rowT), _ptr(edgeT),
                                        _ptr(None if overflow is None else _dev(overflow, "overflow", torch.int32)),
                                        _ptr(max_in_degree), _ptr(ws), ws.numel(), _stream())
    _check(rc, "hc_build_transpose_dev_deg")
    return ptrT, rowT, edgeT


def sample_layers(indptr, indices, seeds, fanout, rng_seed, node_map, emit_view=False, view_edges=False,
                  rng_seed_at=None):
    """Layered neighbour sampling without replacement.  Returns (ptr, idx, sub_to_full, counts) as
    device tensors at their capacity; ``counts`` (int64[2L+2] on the device) holds the node count
    within k hops for k = 0..L and then the cumulative edge count after every hop, so the caller
    slices ptr[:counts[L-1]+1], idx[:counts[2L]], sub_to_full[:counts[L]] once it has read them
    (the last entry is written with ``emit_view`` only: the largest in-degree of a source in the view).
    ``seeds`` must be distinct valid node ids; ``node_map`` comes from ``sample_map`` and is left
    all-unseen again.  Stands where the reference's external loader does
    (/root/reference/hiscache/history_trainer.py:19,26).  ``emit_view=True`` appends (ptrT, rowT, edgeT):
    the transposed view of the whole sampled CSR, built behind the sampling with the sizes still on the
    device (``build_transpose_dev``), for ``BatchView`` once the caller has read ``counts``; edgeT is
    None unless ``view_edges`` (the relational layer's backward reads it).  ``rng_seed_at`` (a one-element
    int64 tensor in device or pinned host memory) replaces ``rng_seed``: the seed is read from it when the
    first kernel runs, which lets a call recorded in a HIP graph be replayed with a new seed."""
    lib = load_library()
    _dev(indptr, "indptr", torch.int64)
    _dev(indices, "indices", torch.int64)
    _dev(seeds, "seeds", torch.int64)
    _dev(node_map, "node_map", torch.int32)
    N = indptr.numel() - 1
    if node_map.numel() < N:
        raise ValueError("node_map is shorter than the graph")
    L = len(fanout)
    n_seed = seeds.numel()
    if n_seed == 0:
        raise ValueError("no seeds")
    fan = (ctypes.c_int64 * L)(*[int(f) for f in fanout])
    rows, edges, nodes = sample_capacity(n_seed, fanout, N)
    dev = seeds.device
    ptr = torch.empty(rows + 1, dtype=torch.int64, device=dev)
    idx = torch.empty(max(edges, 1), dtype=torch.int64, device=dev)
    s2f = torch.empty(max(nodes, 1), dtype=torch.int64, device=dev)
    counts = torch.empty(2 * L + 2, dtype=torch.int64, device=dev)     # (the last entry: see emit_view)
    ws_bytes = int(lib.hc_sample_workspace_bytes(n_seed, ctypes.cast(fan, _c_p), L, N))
    if ws_bytes == 0:
        raise ValueError("unsupported fanout / batch size")
    ws = _workspace(ws_bytes, dev)
    if rng_seed_at is not None:
        if rng_seed_at.dtype != torch.int64 or rng_seed_at.numel() < 1 or not (
                rng_seed_at.is_cuda or rng_seed_at.is_pinned()):
            raise ValueError("rng_seed_at must be an int64 tensor in device or pinned host memory")
        rc = lib.hc_sample_layers_seed_at(_ptr(indptr), _ptr(indices), N, _ptr(seeds), n_seed,
                                          ctypes.cast(fan, _c_p), L, _ptr(rng_seed_at), _ptr(node_map), _ptr(ptr),
                                          _ptr(idx), _ptr(s2f), _ptr(counts), _ptr(ws), ws_bytes, _stream())
    else:
        rc = lib.hc_sample_layers(_ptr(indptr), _ptr(indices), N, _ptr(seeds), n_seed, ctypes.cast(fan, _c_p), L,
                                  ctypes.c_uint64(int(rng_seed) & 0xFFFFFFFFFFFFFFFF), _ptr(node_map), _ptr(ptr),
                                  _ptr(idx), _ptr(s2f), _ptr(counts), _ptr(ws), ws_bytes, _stream())
    _check(rc, "hc_sample_layers")
    if emit_view:
        ptrT, rowT, edgeT = build_transpose_dev(ptr, idx, counts[L - 1:L], counts[2 * L:2 * L + 1],
                                                counts[L:L + 1], edges, nodes, want_edges=view_edges,
                                                max_in_degree=counts[2 * L + 1:])
        return ptr, idx, s2f, counts, ptrT, rowT, edgeT
    return ptr, idx, s2f, counts


def long_row_edges(feature_width, dtype=torch.float32):
    """Rows with more edges than this are summed as four quarters by the mean forward (0: never)."""
    return int(load_library().hc_aggr_fwd_long_row_edges(int(feature_width), _DTYPES[dtype]))


def bwd_chunk_edges(feature_width):
    """Sources with more incoming edges than this are summed in chunks by the mean backward (0: never)."""
    return int(load_library().hc_aggr_bwd_chunk_edges(int(feature_width)))


def version():
    return load_library().hc_version().decode()
