"""ctypes binding of oracle/route_sort.c (plain-C oracle). TEST INFRASTRUCTURE ONLY."""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile the C restatement; force=True compiles also where a built library is there."""
    subprocess.run(["make", "-s"] + (["-B"] if force else []) + ["-C", _HERE, "liboracle_moe.so"], check=True)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle_moe.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def route(logits, k, norm):
    """logits: float array [N, E] -> (idx int32 [N, k], w float32 [N, k])."""
    lg = np.ascontiguousarray(np.asarray(logits, dtype=np.float32))
    N, E = lg.shape
    idx = np.empty((N, k), dtype=np.int32)
    w = np.empty((N, k), dtype=np.float32)
    rc = lib().oracle_route(_p(lg), N, E, k, int(bool(norm)), _p(idx), _p(w))
    if rc:
        raise RuntimeError(f"oracle_route failed ({rc})")
    return idx, w


def sort_by_expert(idx, w, E):
    """idx int32 [N, k], w [N, k] float16 or float32 -> counts, offsets, token, wsorted, pos_of."""
    idx = np.ascontiguousarray(np.asarray(idx, dtype=np.int32))
    w = np.ascontiguousarray(w)
    N, k = idx.shape
    M = N * k
    counts = np.empty(E, dtype=np.int32)
    offsets = np.empty(E + 1, dtype=np.int32)
    token = np.empty(M, dtype=np.int32)
    wsorted = np.empty(M, dtype=w.dtype)
    pos_of = np.empty(M, dtype=np.int32)
    rc = lib().oracle_sort_by_expert(_p(idx), _p(w), w.dtype.itemsize, M, k, E, _p(counts), _p(offsets),
                                     _p(token), _p(wsorted), _p(pos_of))
    if rc:
        raise RuntimeError(f"oracle_sort_by_expert failed ({rc})")
    return counts, offsets, token, wsorted, pos_of


def combine_order(idx):
    idx = np.ascontiguousarray(np.asarray(idx, dtype=np.int32))
    N, k = idx.shape
    order = np.empty((N, k), dtype=np.int32)
    lib().oracle_combine_order(_p(idx), N, k, _p(order))
    return order


def experts_f32(h, idx, w, gate_up, down):
    h = np.ascontiguousarray(h, dtype=np.float32)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    gu = np.ascontiguousarray(gate_up, dtype=np.float32)
    dn = np.ascontiguousarray(down, dtype=np.float32)
    N, H = h.shape
    k = idx.shape[1]
    E, I = dn.shape[0], dn.shape[2]
    out = np.empty((N, H), dtype=np.float32)
    rc = lib().oracle_experts_f32(_p(h), _p(idx), _p(w), _p(gu), _p(dn), N, k, E, H, I, _p(out))
    if rc:
        raise RuntimeError(f"oracle_experts_f32 failed ({rc})")
    return out
