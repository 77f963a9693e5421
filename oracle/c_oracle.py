"""TEST INFRASTRUCTURE ONLY -- ctypes binding of the plain-C checker (oracle/nd_oracle.c)."""

import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libnd_oracle.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", HERE], check=True, capture_output=True)
        h = ctypes.CDLL(LIB)
        h.oracle_nd_rank.restype = ctypes.c_int
        h.oracle_nd_rank.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        h.oracle_crowding.restype = ctypes.c_int
        h.oracle_crowding.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        h.oracle_select.restype = ctypes.c_int
        h.oracle_select.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p,
                                    ctypes.c_void_p, ctypes.c_void_p]
        h.oracle_first_front.restype = ctypes.c_int
        h.oracle_first_front.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        h.oracle_threads.restype = ctypes.c_int
        h.oracle_threads.argtypes = []
        _lib = h
    return _lib


def threads() -> int:
    """Threads that the checker's parallel loops run on."""
    return int(lib().oracle_threads())


def _f32(f):
    return np.ascontiguousarray(np.asarray(f, dtype=np.float32))


def nd_rank(f):
    f = _f32(f)
    rank = np.empty(f.shape[0], dtype=np.int32)
    fronts = lib().oracle_nd_rank(f.ctypes.data, f.shape[0], f.shape[1], rank.ctypes.data)
    if fronts < 0:
        raise MemoryError("oracle_nd_rank")
    return rank, fronts


def crowding(costs, mask):
    c = _f32(costs)
    dist = np.empty(c.shape[0], dtype=np.float32)
    mk = None if mask is None else np.ascontiguousarray(np.asarray(mask, dtype=np.uint8))
    if lib().oracle_crowding(c.ctypes.data, c.shape[0], c.shape[1], None if mk is None else mk.ctypes.data, dist.ctypes.data):
        raise MemoryError("oracle_crowding")
    return dist


def select(f, topk):
    f = _f32(f)
    n = f.shape[0]
    rank = np.empty(n, dtype=np.int32)
    dist = np.empty(n, dtype=np.float32)
    order = np.empty(topk, dtype=np.int64)
    fronts = lib().oracle_select(f.ctypes.data, n, f.shape[1], topk, rank.ctypes.data, dist.ctypes.data, order.ctypes.data)
    if fronts < 0:
        raise RuntimeError(f"oracle_select failed ({fronts})")
    return order, rank, dist, fronts


def first_front(f):
    f = _f32(f)
    mask = np.empty(f.shape[0], dtype=np.uint8)
    lib().oracle_first_front(f.ctypes.data, f.shape[0], f.shape[1], mask.ctypes.data)
    return mask.astype(bool)
