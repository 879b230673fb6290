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


def build_transpose(ptr, idx, n_src, ptrT=None, rowT=None):
    ptr, idx = _arr(ptr, np.int64), _arr(idx, np.int64)
    R = len(ptr) - 1
    if ptrT is None:
        ptrT = np.empty(n_src + 1, np.int64)
    if rowT is None:
        rowT = np.empty(max(int(ptr[R]), 1), np.int32)
    rc = lib().mt_build_transpose(_p(ptr), _p(idx), _I(R), _I(n_src), _p(ptrT), _p(rowT))
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
