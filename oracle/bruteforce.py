"""ctypes binding of ``oracle/bruteforce.c`` (plain-C, double-precision loops).  TEST INFRASTRUCTURE ONLY.

The shared object is built by ``make -C oracle`` (``__graft_entry__.build()`` does it); it is
loaded from ``oracle/_build/libbruteforce.so`` and never built at import time.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libbruteforce.so")
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(f"{_LIB_PATH} missing: run `make -C oracle` (or __graft_entry__.build())")
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("bf_router_topk", "bf_prologue", "bf_expert", "bf_mlp", "bf_bucket", "bf_peer", "bf_pkm"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def router_topk(lp: np.ndarray, nk: int, K: int):
    """lp [2,T,nk] float32 -> (scores [T,K] float32, flat indices [T,K] int64), ties to the lowest index."""
    lp = np.ascontiguousarray(lp, dtype=np.float32)
    T = lp.shape[1]
    scores = np.empty((T, K), np.float32)
    idx = np.empty((T, K), np.int64)
    rc = _load().bf_router_topk(_p(lp), ctypes.c_int64(T), ctypes.c_int(nk), ctypes.c_int(K), _p(scores), _p(idx))
    if rc:
        raise ValueError(f"bf_router_topk failed: {rc}")
    return scores, idx


def prologue(x: np.ndarray, wr: np.ndarray, nk: int, training=True, mean=None, var=None, eps=1e-5):
    """Returns (logits [2,T,nk], lp [2,T,nk], batch mean [H], biased batch var [H]) in float64."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    wr = np.ascontiguousarray(wr, dtype=np.float64)
    T, H = x.shape
    logits = np.empty((2, T, nk), np.float64)
    lp = np.empty((2, T, nk), np.float64)
    m_out = np.empty(H, np.float64)
    v_out = np.empty(H, np.float64)
    m_in = np.ascontiguousarray(mean if mean is not None else np.zeros(H), dtype=np.float64)
    v_in = np.ascontiguousarray(var if var is not None else np.ones(H), dtype=np.float64)
    rc = _load().bf_prologue(_p(x), _p(wr), ctypes.c_int64(T), ctypes.c_int(H), ctypes.c_int(nk),
                             ctypes.c_int(1 if training else 0), _p(m_in), _p(v_in), ctypes.c_double(eps),
                             _p(m_out), _p(v_out), _p(logits), _p(lp))
    if rc:
        raise ValueError(f"bf_prologue failed: {rc}")
    return logits, lp, m_out, v_out


def expert(x, wd, wu, idx, g):
    x, wd, wu, g = (np.ascontiguousarray(a, dtype=np.float64) for a in (x, wd, wu, g))
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    T, H = x.shape
    out = np.empty((T, H), np.float64)
    rc = _load().bf_expert(_p(x), _p(wd), _p(wu), _p(idx), _p(g), ctypes.c_int64(T), ctypes.c_int(H),
                           ctypes.c_int64(wd.shape[0]), ctypes.c_int(idx.shape[1]), _p(out))
    if rc:
        raise ValueError(f"bf_expert failed: {rc}")
    return out


def mlp(x, wg, wu, wd):
    x, wg, wu, wd = (np.ascontiguousarray(a, dtype=np.float64) for a in (x, wg, wu, wd))
    T, H = x.shape
    out = np.empty((T, H), np.float64)
    rc = _load().bf_mlp(_p(x), _p(wg), _p(wu), _p(wd), ctypes.c_int64(T), ctypes.c_int(H),
                        ctypes.c_int(wg.shape[0]), _p(out))
    if rc:
        raise ValueError(f"bf_mlp failed: {rc}")
    return out


def bucket(idx: np.ndarray, num_experts: int):
    """idx [P] int64 -> (expert_offsets [E+1] int32, sorted_pair_ids [offsets[E]] int32) by exhaustive scan."""
    idx = np.ascontiguousarray(idx, dtype=np.int64).reshape(-1)
    offsets = np.empty(num_experts + 1, np.int32)
    pairs = np.empty(max(idx.size, 1), np.int32)
    rc = _load().bf_bucket(_p(idx), ctypes.c_int64(idx.size), ctypes.c_int64(num_experts), _p(offsets), _p(pairs))
    if rc:
        raise ValueError(f"bf_bucket failed: {rc}")
    return offsets, pairs[: offsets[-1]]


def peer(x, wd, wu, idx, g):
    x, wd, wu, g = (np.ascontiguousarray(a, dtype=np.float64) for a in (x, wd, wu, g))
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    T, H = x.shape
    out = np.empty((T, H), np.float64)
    rc = _load().bf_peer(_p(x), _p(wd), _p(wu), _p(idx), _p(g), ctypes.c_int64(T), ctypes.c_int(H),
                         ctypes.c_int64(wd.shape[0]), ctypes.c_int(idx.shape[1]), _p(out))
    if rc:
        raise ValueError(f"bf_peer failed: {rc}")
    return out


def pkm(values, idx, w):
    values, w = (np.ascontiguousarray(a, dtype=np.float64) for a in (values, w))
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    T, H = idx.shape[0], values.shape[1]
    out = np.empty((T, H), np.float64)
    rc = _load().bf_pkm(_p(values), _p(idx), _p(w), ctypes.c_int64(T), ctypes.c_int(H), ctypes.c_int64(values.shape[0]),
                        ctypes.c_int(idx.shape[1]), _p(out))
    if rc:
        raise ValueError(f"bf_pkm failed: {rc}")
    return out
