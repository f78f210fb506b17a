"""numpy-facing wrapper around libck_oracle.so (oracle/ck_oracle.c).

TEST INFRASTRUCTURE ONLY -- the checker, never the product. Build with `python oracle/build.py`.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_int32, c_int64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libck_oracle.so")
_lib = None


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _build

            _build.build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_count.argtypes = [c_void_p, c_int64, c_int32, c_void_p]
        lib.oracle_offsets.argtypes = [c_void_p, c_int32, c_void_p, c_void_p]
        lib.oracle_sort_by_expert.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_void_p]
        lib.oracle_segments.argtypes = [c_void_p, c_void_p, c_int32, c_int32, c_int64, c_void_p, c_void_p, c_void_p]
        lib.oracle_topk_softmax.argtypes = [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p]
        for f in ("oracle_count", "oracle_offsets", "oracle_sort_by_expert", "oracle_segments", "oracle_topk_softmax"):
            getattr(lib, f).restype = None
        _lib = lib
    return _lib


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def count(ids: np.ndarray, num_bins: int) -> np.ndarray:
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    counts = np.empty(num_bins, dtype=np.uint32)
    _load().oracle_count(_p(ids), ids.size, num_bins, _p(counts))
    return counts


def offsets(counts: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """(ends, starts): inclusive and exclusive prefix sums."""
    counts = np.ascontiguousarray(counts, dtype=np.uint32)
    ends = np.empty_like(counts)
    starts = np.empty_like(counts)
    _load().oracle_offsets(_p(counts), counts.size, _p(ends), _p(starts))
    return ends, starts


def sort_by_expert(ids: np.ndarray, num_experts: int) -> tuple[np.ndarray, np.ndarray]:
    """(sorted_expert_idxs, sorted_scattered_idxs) of the stable sort; ids must lie in [0, num_experts)."""
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    assert ids.size == 0 or (ids.min() >= 0 and ids.max() < num_experts)
    se = np.empty(ids.size, dtype=np.int32)
    ss = np.empty(ids.size, dtype=np.int32)
    _load().oracle_sort_by_expert(_p(ids), ids.size, num_experts, _p(se), _p(ss))
    return se, ss


def segments(counts: np.ndarray, sorted_scattered_idxs: np.ndarray, align: int, max_rows: int):
    """(seg_starts [E+1], row_slot [max_rows] with -1 in pad rows, tile_expert [max_rows/align])."""
    counts = np.ascontiguousarray(counts, dtype=np.uint32)
    ss = np.ascontiguousarray(sorted_scattered_idxs, dtype=np.int32)
    E = counts.size
    seg_starts = np.empty(E + 1, dtype=np.int32)
    row_slot = np.empty(max_rows, dtype=np.int32)
    tile_expert = np.empty(max_rows // align, dtype=np.int32)
    _load().oracle_segments(_p(counts), _p(ss), E, align, max_rows, _p(seg_starts), _p(row_slot), _p(tile_expert))
    return seg_starts, row_slot, tile_expert


def topk_softmax(logits: np.ndarray, k: int) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """(selected int32 [T,k], gates fp32 [T,k], values fp32 [T,k]); logits are taken as fp32."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, E = logits.shape
    selected = np.empty((T, k), dtype=np.int32)
    gates = np.empty((T, k), dtype=np.float32)
    values = np.empty((T, k), dtype=np.float32)
    _load().oracle_topk_softmax(_p(logits), T, E, k, _p(selected), _p(gates), _p(values))
    return selected, gates, values
