"""NumPy front end of ``hc_cpu_mt.c``: the aggregation step written for all host cores (OpenMP).

TEST INFRASTRUCTURE ONLY: the benchmark times it as the CPU baseline and the tests check it against
the single-threaded statement in ``hc_oracle.c``; the product package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcpumt.so")
_lib = None


def build(force=False):
    src = os.path.join(_HERE, "hc_cpu_mt.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcpumt.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _I(v):
    return ctypes.c_int64(int(v))


def _arr(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def num_threads():
    return int(lib().mt_num_threads())


def fwd_mean_src(ptr, idx, feat, hmap_src, hist, split_above=0, out=None):
    ptr, idx, feat = _arr(ptr, np.int64), _arr(idx, np.int64), _arr(feat, np.float32)
    R, F = len(ptr) - 1, feat.shape[1]
    hsize = 0
    if hmap_src is not None:
        hmap_src, hist = _arr(hmap_src, np.int64), _arr(hist, np.float32)
        hsize = hist.shape[1]
    if out is None:
        out = np.empty((R, F), np.float32)
    rc = lib().mt_fwd_mean_src(_p(ptr), _p(idx), _p(feat), _p(hmap_src), _p(hist), _p(out), _I(R), _I(F), _I(hsize),
                               _I(split_above))
    if rc != 0:
        raise RuntimeError("mt_fwd_mean_src failed")
    return out


def build_transpose(ptr, idx, n_src, ptrT=None, rowT=None, hmap_src=None):
    ptr, idx = _arr(ptr, np.int64), _arr(idx, np.int64)
    hmap_src = None if hmap_src is None else _arr(hmap_src, np.int64)
    R = len(ptr) - 1
    if ptrT is None:
        ptrT = np.empty(n_src + 1, np.int64)
    if rowT is None:
        rowT = np.empty(max(int(ptr[R]), 1), np.int32)
    rc = lib().mt_build_transpose(_p(ptr), _p(idx), _I(R), _I(n_src), _p(ptrT), _p(rowT), _p(hmap_src))
    if rc != 0:
        raise ValueError("mt_build_transpose: a source id is out of range")
    return ptrT, rowT


def bwd_mean(ptr, ptrT, rowT, g, n_src, chunk=0, out=None):
    ptr, g = _arr(ptr, np.int64), _arr(g, np.float32)
    F = g.shape[1]
    if out is None:
        out = np.empty((n_src, F), np.float32)
    rc = lib().mt_bwd_mean(_p(ptr), _p(ptrT), _p(rowT), _p(g), _p(out), _I(n_src), _I(F), _I(chunk))
    if rc != 0:
        raise RuntimeError("mt_bwd_mean failed")
    return out


def f32_to_f16_bits(x):
    f = lib().mt_f32_to_f16
    f.restype = ctypes.c_uint16
    return np.array([f(ctypes.c_float(float(v))) for v in np.asarray(x, np.float32).ravel()], np.uint16)


def grad_check_f16(grad, emb, slot, age, sub_to_full, thres, age_limit, table, full2slot, slot2full, checkin,
                   header, glb_iter):
    """Fused admission into an fp16 table (uint16 bits), L2 scores, strict ``<``; maps, header and table are
    updated in place.  Returns (mask[bool], score[f32]).  Raises when more rows are admitted than the table
    holds (the sequential statement covers that case)."""
    grad, emb = _arr(grad, np.float32), _arr(emb, np.float32)
    M, F = emb.shape
    slot, sub_to_full = _arr(slot, np.int64), _arr(sub_to_full, np.int64)
    age = None if age is None else _arr(age, np.int32)
    assert table.dtype == np.uint16 and table.flags["C_CONTIGUOUS"] and table.shape[1] == F
    for a in (full2slot, slot2full, header):
        assert a.dtype == np.int64 and a.flags["C_CONTIGUOUS"]
    mask = np.zeros(M, np.uint8)
    score = np.zeros(M, np.float32)
    rank = np.zeros(M, np.int64)
    rc = lib().mt_grad_check_f16(_p(grad), _p(emb), _p(slot), _p(age), _p(sub_to_full), ctypes.c_float(float(thres)),
                                 ctypes.c_int32(int(age_limit)), _p(mask), _p(score), _p(table), _I(table.shape[0]),
                                 _p(full2slot), _p(slot2full), _p(checkin), _p(header), _I(glb_iter), _I(M), _I(F),
                                 _p(rank))
    if rc != 0:
        raise ValueError("mt_grad_check_f16: more admitted rows than table slots")
    return mask.astype(bool), score


def score_rows(grad, hw=True):
    """L2 row scores; ``hw`` selects the build that uses the FMA instruction when the CPU has it."""
    grad = _arr(grad, np.float32)
    out = np.zeros(grad.shape[0], np.float32)
    lib().mt_score_rows(_p(grad), _I(grad.shape[0]), _I(grad.shape[1]), _p(out), ctypes.c_int(int(hw)))
    return out


def convert_row(x, hw=True):
    """fp32 -> fp16 bits of one row; ``hw`` selects the F16C build when the CPU has it."""
    x = _arr(x, np.float32).ravel()
    out = np.zeros(x.size, np.uint16)
    lib().mt_convert_row(_p(x), _p(out), _I(x.size), ctypes.c_int(int(hw)))
    return out
