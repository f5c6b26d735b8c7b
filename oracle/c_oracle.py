"""ctypes binding of oracle/_build/libmoe_oracle.so (moe_oracle.c) — TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_int32, c_int64, c_void_p

import numpy as np


_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "_build", "libmoe_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _DIR], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return _SO


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        for name in ["xo_count", "xo_route", "xo_topk_softmax", "xo_swiglu", "xo_swiglu_bwd", "xo_moe_forward"]:
            getattr(_lib, name).restype = None
    return _lib


def _p(a: np.ndarray) -> c_void_p:
    return a.ctypes.data_as(c_void_p)


def count(ids: np.ndarray, bins: int) -> np.ndarray:
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    out = np.zeros(bins, dtype=np.uint32)
    load().xo_count(_p(ids), c_int64(ids.size), c_int32(bins), _p(out))
    return out


def route(ids: np.ndarray, bins: int):
    """Returns (counts uint32[E], offsets int32[E+1], sorted_ids int64[n], perm int64[n])."""

    ids = np.ascontiguousarray(ids, dtype=np.int64)
    n = ids.size
    counts = np.zeros(bins, dtype=np.uint32)
    offsets = np.zeros(bins + 1, dtype=np.int32)
    sorted_ids = np.zeros(n, dtype=np.int64)
    perm = np.zeros(n, dtype=np.int64)
    load().xo_route(_p(ids), c_int64(n), c_int32(bins), _p(counts), _p(offsets), _p(sorted_ids), _p(perm))
    return counts, offsets, sorted_ids, perm


def topk_softmax(logits: np.ndarray, k: int):
    """logits float32 [T, E] -> (weights float64 [T, k], idx int64 [T, k])."""

    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, E = logits.shape
    weights = np.zeros((T, k), dtype=np.float64)
    idx = np.zeros((T, k), dtype=np.int64)
    load().xo_topk_softmax(_p(logits), c_int64(T), c_int32(E), c_int32(k), _p(weights), _p(idx))
    return weights, idx


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    gate = np.ascontiguousarray(gate, dtype=np.float64)
    up = np.ascontiguousarray(up, dtype=np.float64)
    y = np.zeros_like(gate)
    load().xo_swiglu(_p(gate), _p(up), c_int64(gate.size), _p(y))
    return y


def swiglu_bwd(gate: np.ndarray, up: np.ndarray, dy: np.ndarray):
    gate = np.ascontiguousarray(gate, dtype=np.float64)
    up = np.ascontiguousarray(up, dtype=np.float64)
    dy = np.ascontiguousarray(dy, dtype=np.float64)
    dg, du = np.zeros_like(gate), np.zeros_like(gate)
    load().xo_swiglu_bwd(_p(gate), _p(up), _p(dy), c_int64(gate.size), _p(dg), _p(du))
    return dg, du


def moe_forward(x, w1, w2, weights, idx) -> np.ndarray:
    """Token-by-token SwiGLU MoE forward in float64.  x [T,H], w1 [E,2I,H], w2 [E,H,I]."""

    x = np.ascontiguousarray(x, dtype=np.float64)
    w1 = np.ascontiguousarray(w1, dtype=np.float64)
    w2 = np.ascontiguousarray(w2, dtype=np.float64)
    weights = np.ascontiguousarray(weights, dtype=np.float64)
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    T, H = x.shape
    I = w2.shape[2]
    k = idx.shape[1]
    y = np.zeros((T, H), dtype=np.float64)
    load().xo_moe_forward(_p(x), _p(w1), _p(w2), _p(weights), _p(idx), c_int64(T), c_int32(H), c_int32(I), c_int32(k), _p(y))
    return y
