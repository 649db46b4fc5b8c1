"""ctypes access to the plain-C oracle (oracle/acache_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import c_float, c_int32, c_int64, c_void_p
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "liboracle.so"


def build() -> Path:
    subprocess.run(["make", "-s", "-C", str(HERE), "-B", "liboracle.so"], check=True)
    return LIB


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            build()
        _lib = ctypes.CDLL(str(LIB))
    return _lib


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(c_void_p)


def rope_table(rows: int, D: int, theta: float):
    cos = np.empty((rows, D), np.float32)
    sin = np.empty((rows, D), np.float32)
    load().oracle_rope_table(_p(cos), _p(sin), c_int32(rows), c_int32(D), c_float(theta))
    return cos, sin


def relocate_rope_gather(k_cache, v_cache, slot, delta, cos, sin, dtype_code: int):
    """Caches: numpy ``[L, S, H, D]`` (uint16 for bf16, float32 for fp32)."""
    L, S, H, D = k_cache.shape
    T = slot.shape[0]
    out_k = np.empty((L, T, H, D), k_cache.dtype)
    out_v = np.empty((L, T, H, D), k_cache.dtype)
    rope_rows = 0 if cos is None else cos.shape[0]
    load().oracle_relocate_rope_gather(
        _p(out_k), _p(out_v), _p(np.ascontiguousarray(k_cache)), _p(np.ascontiguousarray(v_cache)),
        _p(slot.astype(np.int32)), _p(None if delta is None else delta.astype(np.int32)),
        _p(cos), _p(sin), c_int64(T), c_int32(L), c_int32(H), c_int32(D), c_int32(dtype_code),
        c_int64(S), c_int32(rope_rows), c_int64(S * H * D), c_int64(T * H * D))
    return out_k, out_v


def kv_scatter(k_cache, v_cache, key, value, slot, dtype_code: int):
    S, H, D = k_cache.shape
    load().oracle_kv_scatter(_p(k_cache), _p(v_cache), _p(np.ascontiguousarray(key)),
                             _p(np.ascontiguousarray(value)), _p(slot.astype(np.int32)),
                             c_int64(key.shape[0]), c_int32(H), c_int32(D), c_int32(dtype_code), c_int64(S))


def topk(scores: np.ndarray, k: int, largest: bool = True):
    scores = np.ascontiguousarray(scores, np.float32)
    k = min(k, scores.shape[0])
    out = np.empty(k, np.int32)
    load().oracle_topk(_p(out), _p(scores), c_int32(scores.shape[0]), c_int32(k), c_int32(1 if largest else 0))
    return out


def dense_attention(q, k, v, scale: float):
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    Tq, H, D = q.shape
    Tk, Hkv, _ = k.shape
    out = np.empty_like(q)
    load().oracle_dense_attention(_p(out), _p(q), _p(k), _p(v), c_int32(Tq), c_int32(Tk), c_int32(H),
                                  c_int32(Hkv), c_int32(D), c_float(scale))
    return out
