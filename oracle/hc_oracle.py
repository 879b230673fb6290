"""NumPy front end of the CPU oracle (``hc_oracle.c``).

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the benchmark's CPU
baseline leg may import this module; the product package never does.

Every function takes and returns NumPy arrays (int64 indices, fp32 data) and
calls the plain-C restatement of the reference semantics.  The C file cites the
reference lines each routine follows.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liborc.so")

NORM_L2, NORM_L1 = 0, 1
CMP_LT, CMP_NOT_GT = 0, 1
DT_F32, DT_F16, DT_BF16 = 0, 1, 2


def build(force=False):
    """Compile ``hc_oracle.c`` with gcc (a one-file build, about a second)."""
    src = os.path.join(_HERE, "hc_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liborc.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_row_score.restype = ctypes.c_float
        _lib.orc_f16_to_f32.restype = ctypes.c_float
        _lib.orc_bf16_to_f32.restype = ctypes.c_float
        _lib.orc_f32_to_f16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
    return _lib


def _p(a):
    if a is None:
        return ctypes.c_void_p(None)
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    # data_as keeps a reference to the array, so a converted temporary (``_p(_u8(mask))``) stays
    # alive until the C call that receives the pointer has returned
    return a.ctypes.data_as(ctypes.c_void_p)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return None if a is None else np.ascontiguousarray(a).astype(np.uint8)


def _I(v):
    return ctypes.c_int64(int(v))


def _check(rc, name):
    if rc != 0:
        raise ValueError(f"oracle {name} rejected its input (code {rc})")


# --------------------------------------------------------------------------- aggregation
def fwd_mean_row(ptr, idx, vin, hmap, hbuf, num_node=None, split_above=0):
    ptr, idx, vin = _i64(ptr), _i64(idx), _f32(vin)
    R = len(ptr) - 1 if not num_node else int(num_node)
    F = vin.shape[-1]
    hsize = 0
    if hmap is not None:
        hmap, hbuf = _i64(hmap), _f32(hbuf)
        hsize = hbuf.shape[-1] if hbuf.ndim == 2 else F
    out = np.zeros((R, F), np.float32)
    _check(lib().orc_fwd_mean_row(_p(ptr), _p(idx), _p(vin), _p(hmap), _p(hbuf), _p(out),
                                  _I(R), _I(F), _I(hsize), _I(split_above)), "fwd_mean_row")
    return out


def fwd_edge_value(ptr, idx, ev, vin, hmap, hbuf, num_node=None, split_above=0):
    ptr, idx, vin, ev = _i64(ptr), _i64(idx), _f32(vin), _f32(ev)
    R = len(ptr) - 1 if not num_node else int(num_node)
    if ev.ndim == 2:
        H, F = vin.shape[1], vin.shape[2]
        hsize = 0
        if hmap is not None:
            hmap, hbuf = _i64(hmap), _f32(hbuf)
            hsize = hbuf.shape[-1]
        out = np.zeros((R, H, F), np.float32)
        _check(lib().orc_fwd_edge_value_multi_head(_p(ptr), _p(idx), _p(ev), _p(vin), _p(hmap),
                                                   _p(hbuf), _p(out), _I(R), _I(F), _I(hsize), _I(H)),
               "fwd_edge_value_multi_head")
        return out
    F = vin.shape[-1]
    hsize = 0
    if hmap is not None:
        hmap, hbuf = _i64(hmap), _f32(hbuf)
        hsize = hbuf.shape[-1]
    out = np.zeros((R, F), np.float32)
    _check(lib().orc_fwd_edge_value(_p(ptr), _p(idx), _p(ev), _p(vin), _p(hmap), _p(hbuf), _p(out),
                                    _I(R), _I(F), _I(hsize), _I(split_above)), "fwd_edge_value")
    return out


def fwd_mean_src(ptr, idx, feat, hmap_src, hist, num_node=None, split_above=0):
    ptr, idx, feat = _i64(ptr), _i64(idx), _f32(feat)
    R = len(ptr) - 1 if not num_node else int(num_node)
    F = feat.shape[-1]
    hsize = 0
    if hmap_src is not None:
        hmap_src, hist = _i64(hmap_src), _f32(hist)
        hsize = hist.shape[-1]
    out = np.zeros((R, F), np.float32)
    _check(lib().orc_fwd_mean_src(_p(ptr), _p(idx), _p(feat), _p(hmap_src), _p(hist), _p(out),
                                  _I(R), _I(F), _I(hsize), _I(split_above)), "fwd_mean_src")
    return out


def bwd_mean_row(ptr, idx, g, hmap, n_src, hbuf_shape=None, chunk=0):
    """Returns (grad_input[n_src,F], grad_history[R,hsize] or None)."""
    ptr, idx, g = _i64(ptr), _i64(idx), _f32(g)
    R, F = g.shape
    gout = np.zeros((n_src, F), np.float32)
    ghist = None
    hsize = 0
    if hmap is not None:
        hmap = _i64(hmap)
        hsize = hbuf_shape[-1] if hbuf_shape is not None else F
        ghist = np.zeros((R, hsize), np.float32)
    _check(lib().orc_bwd_mean_row(_p(ptr), _p(idx), _p(g), _p(hmap), _p(gout), _p(ghist),
                                  _I(R), _I(F), _I(hsize), _I(n_src), _I(chunk)), "bwd_mean_row")
    return gout, ghist


def bwd_mean_row_batch_view(ptr, idx, g, hmap, n_src, view_rows, hbuf_shape=None, chunk=0):
    """bwd_mean_row in the summation order of hc_aggr_bwd_batch_view: (ptr, idx) is the whole
    mini-batch CSR (at least ``view_rows`` rows, over which the shared view was built), g [R, F] and
    hmap belong to the layer's first R rows."""
    ptr, idx, g = _i64(ptr), _i64(idx), _f32(g)
    R, F = g.shape
    gout = np.zeros((n_src, F), np.float32)
    ghist = None
    hsize = 0
    if hmap is not None:
        hmap = _i64(hmap)
        hsize = hbuf_shape[-1] if hbuf_shape is not None else F
        ghist = np.zeros((R, hsize), np.float32)
    _check(lib().orc_bwd_mean_row_batch_view(_p(ptr), _p(idx), _p(g), _p(hmap), _p(gout), _p(ghist),
                                             _I(R), _I(F), _I(hsize), _I(n_src), _I(chunk),
                                             _I(view_rows)), "bwd_mean_row_batch_view")
    return gout, ghist


def bwd_mean_src(ptr, idx, g, n_src, chunk=0, hmap_src=None, hist_shape=None):
    """Backward of the mean with per-source substitution.  Without ``hmap_src``: the gradient of the
    row that was read for every source, whichever table it came from.  With ``hmap_src``: returns
    (grad_feat, grad_hist) -- a substituted source s leaves grad_feat[s] = 0 (feat[s] was not read) and
    adds its sum to grad_hist[hmap_src[s]] (sources that share a table row are added in ascending
    source order); ``hist_shape`` None skips grad_hist."""
    all_src = bwd_mean_row(ptr, idx, g, None, n_src, chunk=chunk)[0]
    if hmap_src is None:
        return all_src
    hmap_src = _i64(hmap_src)[:n_src]
    sub = hmap_src != -1
    grad_feat = all_src.copy()
    grad_feat[sub] = 0.0
    grad_hist = None
    if hist_shape is not None:
        grad_hist = np.zeros(hist_shape, np.float32)
        F = all_src.shape[1]
        for s in np.nonzero(sub)[0]:
            grad_hist[hmap_src[s], :F] += all_src[s]
    return grad_feat, grad_hist


def bwd_edge_value(ptr, idx, ev, g, hmap, vin, n_src, hsize=None, want_edge_grad=False):
    """Returns (grad_input, grad_history or None, edge_grad or None)."""
    ptr, idx, ev, g = _i64(ptr), _i64(idx), _f32(ev), _f32(g)
    E = len(idx)
    vin = _f32(vin) if vin is not None else None
    if ev.ndim == 2:
        R, H, F = g.shape
        hs = 0
        ghist = None
        if hmap is not None:
            hmap = _i64(hmap)
            hs = int(hsize)
            ghist = np.zeros((R, hs), np.float32)
        gout = np.zeros((n_src, H, F), np.float32)
        eg = np.zeros((E, H), np.float32) if want_edge_grad else None
        _check(lib().orc_bwd_edge_value_multi_head(_p(ptr), _p(idx), _p(ev), _p(g), _p(hmap), _p(vin),
                                                   _p(gout), _p(ghist), _p(eg), _I(R), _I(F), _I(hs),
                                                   _I(H), _I(n_src), _I(E)), "bwd_edge_value_multi_head")
        return gout, ghist, eg
    R, F = g.shape
    hs = 0
    ghist = None
    if hmap is not None:
        hmap = _i64(hmap)
        hs = int(hsize) if hsize else F
        ghist = np.zeros((R, hs), np.float32)
    gout = np.zeros((n_src, F), np.float32)
    eg = np.zeros((E,), np.float32) if want_edge_grad else None
    _check(lib().orc_bwd_edge_value(_p(ptr), _p(idx), _p(ev), _p(g), _p(hmap), _p(vin), _p(gout),
                                    _p(ghist), _p(eg), _I(R), _I(F), _I(hs), _I(n_src), _I(E)),
           "bwd_edge_value")
    return gout, ghist, eg


def build_transpose(ptr, idx, hmap_row, n_src, num_node=None):
    """Stable CSC view: (ptrT[n_src+1], rowT[E_kept], edgeT[E_kept])."""
    ptr, idx = _i64(ptr), _i64(idx)
    R = len(ptr) - 1 if not num_node else int(num_node)
    hm = _i64(hmap_row) if hmap_row is not None else None
    E = int(ptr[R])
    ptrT = np.zeros(n_src + 1, np.int64)
    rowT = np.zeros(max(E, 1), np.int32)
    edgeT = np.zeros(max(E, 1), np.int32)
    _check(lib().orc_build_transpose(_p(ptr), _p(idx), _p(hm), _I(R), _I(n_src), _p(ptrT), _p(rowT),
                                     _p(edgeT)), "build_transpose")
    k = int(ptrT[n_src])
    return ptrT, rowT[:k].copy(), edgeT[:k].copy()


# --------------------------------------------------------------------------- used masks
def count_history_reconstruct(ptr, idx, history_map, num_node, num_seed, num_layer):
    """Returns a list of num_layer+1 bool arrays of size num_node (reference order)."""
    ptr, idx = _i64(ptr), _i64(idx)
    hm = _i64(history_map) if history_map is not None else None
    L = int(num_layer)
    masks = np.zeros((L + 1, int(num_node)), np.uint8)
    _check(lib().orc_count_history(_p(ptr), _p(idx), _p(hm), _I(0 if hm is None else len(hm)),
                                   _p(masks), _I(len(ptr) - 1), _I(num_node), _I(num_seed),
                                   ctypes.c_int(L)), "count_history")
    return [masks[i].astype(bool) for i in range(L + 1)]


# --------------------------------------------------------------------------- admission
def row_scores(grad, norm_kind=NORM_L2):
    grad = _f32(grad)
    M, F = grad.shape
    out = np.zeros(M, np.float32)
    lib().orc_row_scores(_p(grad), _p(out), _I(M), _I(F), ctypes.c_int(norm_kind))
    return out


def record_history(buffer_new, buffer_all, used_mask, sub_to_full, sub_to_history, history_to_full,
                   full_to_history, header, score, thres, checkin_iter, glb_iter):
    """In-place on buffer_all / history_to_full / full_to_history / header / checkin_iter
    (all NumPy arrays of the reference dtypes).  Returns the admitted mask."""
    for a, dt in ((buffer_all, np.float32), (history_to_full, np.int64), (full_to_history, np.int64),
                  (header, np.int64), (checkin_iter, np.int64)):
        assert a.dtype == dt and a.flags["C_CONTIGUOUS"]
    buffer_new = _f32(buffer_new)
    M = buffer_new.shape[0]
    mask = np.zeros(M, np.uint8)
    thres = np.asarray(thres, np.float32).reshape(1)
    _check(lib().orc_record_history(_p(buffer_new), _p(buffer_all), _p(_u8(used_mask)),
                                    _p(_i64(sub_to_full)), _p(_i64(sub_to_history)),
                                    _p(history_to_full), _p(full_to_history), _p(header),
                                    _p(_f32(score)), _p(thres), _p(checkin_iter), _I(glb_iter), _I(M),
                                    _I(buffer_all.shape[0]), _I(buffer_all.shape[1]), _p(mask)),
           "record_history")
    return mask.astype(bool)


def grad_check(grad, emb, slot, age, used, sub_to_full, thres, age_limit, norm_kind, cmp_kind, table,
               table_dtype, full2slot, slot2full, checkin, header, glb_iter, score_in=None):
    """Fused admission.  `table` is a NumPy array viewed as fp32 or uint16 (fp16/bf16 bits);
    maps/header are int64 arrays updated in place.
    Returns (mask[bool], score[f32], slot_of_row[int64, -1 when not admitted])."""
    emb = _f32(emb)
    M, F = emb.shape
    grad = _f32(grad) if grad is not None else None
    score_in = _f32(score_in) if score_in is not None else None
    mask = np.zeros(M, np.uint8)
    score = np.zeros(M, np.float32)
    slot_out = np.zeros(M, np.int64)
    age = np.ascontiguousarray(age, np.int32) if age is not None else None
    assert table.flags["C_CONTIGUOUS"]
    _check(lib().orc_grad_check(_p(grad), _p(score_in), _p(emb), _p(_i64(slot)), _p(age), _p(_u8(used)),
                                _p(_i64(sub_to_full)), ctypes.c_float(float(thres)),
                                ctypes.c_int32(int(age_limit)), ctypes.c_int(norm_kind),
                                ctypes.c_int(cmp_kind), _p(mask), _p(score), _p(table),
                                ctypes.c_int(table_dtype), _I(table.shape[0]), _p(full2slot),
                                _p(slot2full), _p(checkin), _p(header), _I(glb_iter), _I(M), _I(F),
                                _p(slot_out)), "grad_check")
    return mask.astype(bool), score, slot_out


# --------------------------------------------------------------------------- helpers
def count_num(arr, mmax):
    arr = _i64(arr)
    out = np.zeros(int(mmax) + 1, np.int32)
    _check(lib().orc_count_num(_p(arr), _I(len(arr)), _I(mmax), _p(out)), "count_num")
    return out


def typed_csr(ptr, idx, edge_types, num_rel, num_node, n_src, used_mask=None):
    """(ptr2, idx2[:ptr2[-1]], cnt[num_node, num_rel], deg) of the (row, relation) grouping."""
    ptr, idx, et = _i64(ptr), _i64(idx), _i64(edge_types)
    R, K = int(num_node), int(num_rel)
    E = min(len(idx), len(et))
    used = None if used_mask is None else np.ascontiguousarray(used_mask, dtype=np.uint8)
    ptr2 = np.zeros(R * K + 1, np.int64)
    idx2 = np.zeros(max(E, 1), np.int64)
    cnt = np.zeros(R * K, np.int64)
    deg = np.zeros(R, np.int64)
    _check(lib().orc_typed_csr(_p(ptr), _p(idx), _p(et), _p(used) if used is not None else None, _I(R), _I(E),
                               _I(n_src), ctypes.c_int(K), _p(ptr2), _p(idx2), _p(cnt), _p(deg)), "typed_csr")
    return ptr2, idx2[:ptr2[-1]], cnt.reshape(R, K), deg


def bwd_typed_batch_view(ptr, idx, edge_types, num_rel, g, n_src, used_mask=None):
    """Input gradient of the relational layer, rows and edge slots walked in ascending order
    (hc_aggr_bwd_batch_view_typed); g is [R * num_rel, F]."""
    ptr, idx, et, g = _i64(ptr), _i64(idx), _i64(edge_types), _f32(g)
    K = int(num_rel)
    R, F = g.shape[0] // K, g.shape[1]
    E = min(len(idx), len(et))
    used = None if used_mask is None else np.ascontiguousarray(used_mask, dtype=np.uint8)
    out = np.zeros((n_src, F), np.float32)
    _check(lib().orc_bwd_typed_batch_view(_p(ptr), _p(idx), _p(et), _p(used) if used is not None else None,
                                          _p(g), _p(out), _I(R), _I(E), _I(F), ctypes.c_int(K), _I(n_src)),
           "bwd_typed_batch_view")
    return out


def typed_csr_weights(ptr2, deg, num_rel):
    """The edge weights hc_typed_csr writes beside idx2: fp32 1/deg of the edge's row (deg counts every
    edge of the row, kept or dropped)."""
    ptr2, deg = _i64(ptr2), _i64(deg)
    per_group = np.repeat(np.float32(1.0) / np.maximum(deg, 1).astype(np.float32), int(num_rel))
    return np.repeat(per_group, np.diff(ptr2)).astype(np.float32)


def edge_types_by_ranges(ptr, idx, sub_to_full, num_node, bounds, pair_to_rel):
    """Relation per edge from the node types of its ends (numpy statement; type = number of bounds
    the full id has reached).  -1 outside the first ``num_node`` rows and for sources out of range.
    Stand-in for cxgnncomp_backend.gen_edge_type_mag240m (history_model.py:356): PARITY UNPINNED
    against that library, which is not part of the reference repository."""
    ptr, idx, s2f = _i64(ptr), _i64(idx), _i64(sub_to_full)
    bounds = _i64(bounds)
    table = np.asarray(pair_to_rel, np.int64).reshape(len(bounds) + 1, len(bounds) + 1)
    R = int(num_node)
    out = np.full(len(idx), -1, np.int64)
    end = min(int(ptr[R]), len(idx))
    e = np.arange(end)
    row = np.searchsorted(ptr[1:R + 1], e, side="right")
    src = idx[:end]
    ok = (src >= 0) & (src < len(s2f))
    t_dst = np.searchsorted(bounds, s2f[row], side="right")
    t_src = np.searchsorted(bounds, s2f[np.where(ok, src, 0)], side="right")
    out[:end] = np.where(ok, table[t_dst, t_src], -1)
    return out


def get_graph_structure_score(ptr, idx, num_node, num_seed, num_layer):
    ptr, idx = _i64(ptr), _i64(idx)
    out = np.zeros(int(num_node), np.int64)
    _check(lib().orc_structure_score(_p(ptr), _p(idx), _I(len(ptr) - 1), _I(num_node), _I(num_seed),
                                     ctypes.c_int(int(num_layer)), _p(out)), "structure_score")
    return out


def gather_rows(table, ids, mask=None):
    table = _f32(table)
    ids = _i64(ids)
    out = np.zeros((len(ids), table.shape[1]), np.float32)
    _check(lib().orc_gather_rows(_p(table), _I(table.shape[0]), _p(ids), _p(_u8(mask)), _p(out),
                                 _I(len(ids)), _I(table.shape[1])), "gather_rows")
    return out


def f32_to_f16_bits(x):
    x = _f32(x).ravel()
    return np.array([lib().orc_f32_to_f16(ctypes.c_float(v)) for v in x], np.uint16)


def f32_to_bf16_bits(x):
    x = _f32(x).ravel()
    return np.array([lib().orc_f32_to_bf16(ctypes.c_float(v)) for v in x], np.uint16)


# --------------------------------------------------------------------------- sampler
def mix64(z):
    f = lib().orc_mix64
    f.restype = ctypes.c_uint64
    return int(f(ctypes.c_uint64(int(z) & 0xFFFFFFFFFFFFFFFF)))


def sample_perm(j, d, key):
    f = lib().orc_sample_perm
    f.restype = ctypes.c_uint64
    return int(f(ctypes.c_uint64(int(j)), ctypes.c_uint64(int(d)), ctypes.c_uint64(int(key) & 0xFFFFFFFFFFFFFFFF)))


def sample_layers(indptr, indices, seeds, fanout, rng_seed):
    """Sequential statement of the layered sampler.  Returns a dict with ptr, idx, sub_to_full,
    num_node_in_layer, num_edge_in_layer (NumPy int64), trimmed to their real sizes."""
    indptr, indices, seeds = _i64(indptr), _i64(indices), _i64(seeds)
    fan = _i64(np.asarray(fanout))
    L, n0 = len(fan), len(seeds)
    rows, edges, nodes = 0, 0, n0
    r = n0
    for f in fan:
        rows += r
        edges += r * int(f)
        r = r * int(f)
        nodes += r
    N = len(indptr) - 1
    nodes = min(nodes, max(N, n0))
    ptr = np.zeros(rows + 1, np.int64)
    idx = np.zeros(max(edges, 1), np.int64)
    s2f = np.zeros(nodes, np.int64)
    counts = np.zeros(2 * L + 1, np.int64)
    _check(lib().orc_sample_layers(_p(indptr), _p(indices), _I(N), _p(seeds), _I(n0), _p(fan), ctypes.c_int(L),
                                   ctypes.c_uint64(int(rng_seed) & 0xFFFFFFFFFFFFFFFF), _p(ptr), _p(idx), _p(s2f),
                                   _p(counts)), "sample_layers")
    nnl = counts[:L + 1].copy()
    nel = counts[L + 1:].copy()
    return {"ptr": ptr[: nnl[L - 1] + 1].copy(), "idx": idx[: nel[-1]].copy(), "sub_to_full": s2f[: nnl[L]].copy(),
            "num_node_in_layer": nnl, "num_edge_in_layer": nel}

