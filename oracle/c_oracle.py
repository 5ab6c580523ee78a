"""ctypes loader for the C part of the CPU oracle (fcfs_dispatch.c).

TEST INFRASTRUCTURE ONLY; never imported by the product package.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_fcfs.so")
_lib = None


def build() -> str:
    subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_fcfs_dispatch.restype = ctypes.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def fcfs_dispatch(idx: np.ndarray, num_experts: int, cap: int):
    """idx [T,k] integer array -> (token_map [E,C], slot [T*k], hist [E], kept [E], dropped)."""
    lib = _load()
    T, k = idx.shape
    flat = np.ascontiguousarray(idx, dtype=np.int32).reshape(-1)
    token_map = np.empty((num_experts, max(cap, 0)), dtype=np.int32)
    slot = np.empty(T * k, dtype=np.int32)
    hist = np.empty(num_experts, dtype=np.int32)
    kept = np.empty(num_experts, dtype=np.int32)
    dropped = lib.oracle_fcfs_dispatch(_p(flat), ctypes.c_int64(T), ctypes.c_int32(k),
                                       ctypes.c_int32(num_experts), ctypes.c_int32(cap),
                                       _p(token_map), _p(slot), _p(hist), _p(kept))
    if dropped < 0:
        raise ValueError("expert id out of range")
    return token_map, slot, hist, kept, int(dropped)


def combine_f32(expert_out: np.ndarray, token_map: np.ndarray, w: np.ndarray, T: int, k: int):
    lib = _load()
    E, C, H = expert_out.shape
    eo = np.ascontiguousarray(expert_out, dtype=np.float32)
    tm = np.ascontiguousarray(token_map, dtype=np.int32)
    ww = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    out = np.empty((T, H), dtype=np.float32)
    lib.oracle_combine_f32(_p(eo), _p(tm), _p(ww), ctypes.c_int64(T), ctypes.c_int32(k),
                           ctypes.c_int32(E), ctypes.c_int32(C), ctypes.c_int32(H), _p(out))
    return out
