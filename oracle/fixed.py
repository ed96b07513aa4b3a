"""numpy front-end of the fixed-order C oracle (``pqhsa_oracle.c``).  TEST INFRASTRUCTURE.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
use this module, and only as the checker.
"""

from __future__ import annotations

import ctypes
import math
import os

import numpy as np

from . import build as _build

_LIB = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = _build.LIB
        if not os.path.exists(path):
            path = _build.build()
        _LIB = ctypes.CDLL(path)
        _LIB.pqo_encode.restype = ctypes.c_int
        _LIB.pqo_lut_build.restype = ctypes.c_int
        _LIB.pqo_topk.restype = ctypes.c_int
        _LIB.pqo_attend.restype = ctypes.c_int
    return _LIB


def _c(a: np.ndarray, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _p(a: np.ndarray, ptype):
    return a.ctypes.data_as(ptype)


def resolve_topk(n: int, fraction: float) -> int:
    """k = min(max(ceil(n * fraction), 0), n) — pq_hsa/attention/sparse_attention.py:1779-1783."""
    return min(max(int(math.ceil(n * fraction)), 0), n)


def encode(keys, coarse, codebooks, eps: float = 1e-12):
    keys = _c(keys, np.float32)
    coarse = _c(coarse, np.float32)
    codebooks = _c(codebooks, np.float32)
    n, dim = keys.shape
    num_lists = coarse.shape[0]
    m = codebooks.shape[0]
    norms = np.empty(n, np.float32)
    lists = np.empty(n, np.uint16)
    codes = np.empty(n, np.uint32)
    rc = lib().pqo_encode(_p(keys, _f32p), ctypes.c_int64(n), dim, _p(coarse, _f32p), num_lists,
                          _p(codebooks, _f32p), m, ctypes.c_float(eps), _p(norms, _f32p),
                          _p(lists, _u16p), _p(codes, _u32p))
    if rc != 0:
        raise ValueError(f"pqo_encode failed: {rc}")
    return norms, lists, codes


def value_summaries(values, list_ids, num_lists: int):
    values = _c(values, np.float32)
    list_ids = _c(list_ids, np.uint16)
    n, dv = values.shape
    sums = np.empty((num_lists, dv), np.float32)
    counts = np.empty(num_lists, np.float32)
    vbar = np.empty((num_lists, dv), np.float32)
    lib().pqo_value_summaries(_p(values, _f32p), _p(list_ids, _u16p), ctypes.c_int64(n), dv,
                              num_lists, _p(sums, _f32p), _p(counts, _f32p), _p(vbar, _f32p))
    return sums, counts, vbar


def value_append(value, list_id: int, sums, counts, vbar) -> None:
    value = _c(value, np.float32)
    lib().pqo_value_append(_p(value, _f32p), int(list_id), value.shape[0], _p(sums, _f32p),
                           _p(counts, _f32p), _p(vbar, _f32p))


def lut_build(queries, coarse, codebooks, eps: float = 1e-12):
    queries = _c(queries, np.float32)
    coarse = _c(coarse, np.float32)
    codebooks = _c(codebooks, np.float32)
    g, dim = queries.shape
    num_lists = coarse.shape[0]
    m = codebooks.shape[0]
    qnorm = np.empty(g, np.float32)
    lut = np.empty((g, m, 16), np.float32)
    list_scores = np.empty((g, num_lists), np.float32)
    rc = lib().pqo_lut_build(_p(queries, _f32p), g, dim, _p(coarse, _f32p), num_lists,
                             _p(codebooks, _f32p), m, ctypes.c_float(eps), _p(qnorm, _f32p),
                             _p(lut, _f32p), _p(list_scores, _f32p))
    if rc != 0:
        raise ValueError(f"pqo_lut_build failed: {rc}")
    return qnorm, lut, list_scores


def scan(codes, list_ids, norms, lut, list_scores, qnorm, scale: float):
    codes = _c(codes, np.uint32)
    list_ids = _c(list_ids, np.uint16)
    norms = _c(norms, np.float32)
    lut = _c(lut, np.float32)
    list_scores = _c(list_scores, np.float32)
    qnorm = _c(qnorm, np.float32)
    n = codes.shape[0]
    g, m, _ = lut.shape
    num_lists = list_scores.shape[1]
    logits = np.empty((g, n), np.float32)
    lib().pqo_scan(_p(codes, _u32p), _p(list_ids, _u16p), _p(norms, _f32p), ctypes.c_int64(n),
                   _p(lut, _f32p), _p(list_scores, _f32p), _p(qnorm, _f32p), g, num_lists, m,
                   ctypes.c_float(scale), _p(logits, _f32p))
    return logits


def topk(logits, k: int):
    logits = _c(logits, np.float32)
    squeeze = logits.ndim == 1
    rows = logits.reshape(-1, logits.shape[-1])
    idx = np.empty((rows.shape[0], k), np.int32)
    val = np.empty((rows.shape[0], k), np.float32)
    for r in range(rows.shape[0]):
        rc = lib().pqo_topk(_p(rows[r], _f32p), ctypes.c_int64(rows.shape[1]), k, _p(idx[r], _i32p),
                            _p(val[r], _f32p))
        if rc != 0:
            raise ValueError(f"pqo_topk failed: {rc}")
    if squeeze:
        return idx[0], val[0]
    return idx, val


def attend(queries, keys, values, sink_end: int, logits, topk_idx, list_ids, vbar, scale: float):
    queries = _c(queries, np.float32)
    keys = _c(keys, np.float32)
    values = _c(values, np.float32)
    logits = _c(logits, np.float32)
    topk_idx = _c(topk_idx, np.int32)
    list_ids = _c(list_ids, np.uint16)
    vbar = _c(vbar, np.float32)
    g, dim = queries.shape
    length, dv = values.shape
    n = logits.shape[1]
    k = topk_idx.shape[1]
    out = np.empty((g, dv), np.float32)
    rc = lib().pqo_attend(_p(queries, _f32p), g, dim, dv, _p(keys, _f32p), _p(values, _f32p),
                          ctypes.c_int64(length), int(sink_end), ctypes.c_int64(n),
                          _p(logits, _f32p), _p(topk_idx, _i32p), k, _p(list_ids, _u16p),
                          _p(vbar, _f32p), vbar.shape[0], ctypes.c_float(scale), _p(out, _f32p))
    if rc != 0:
        raise ValueError(f"pqo_attend failed: {rc}")
    return out


def paged_gather(cache_bits, strides, dim: int, block_size: int, block_table, head: int, positions):
    """cache_bits: flat uint16 view of a 16-bit paged cache; strides = (block, row, head) in elements."""
    cache_bits = _c(cache_bits, np.uint16).reshape(-1)
    block_table = _c(block_table, np.int32)
    positions = _c(positions, np.int64)
    out = np.empty((positions.shape[0], dim), np.uint16)
    lib().pqo_paged_gather(_p(cache_bits, _u16p), ctypes.c_int64(strides[0]), ctypes.c_int64(strides[1]),
                           ctypes.c_int64(strides[2]), dim, block_size, _p(block_table, _i32p), head,
                           _p(positions, _i64p), ctypes.c_int64(positions.shape[0]), _p(out, _u16p))
    return out


def decode_step(queries, keys, values, index, *, sink: int, local: int, fraction: float, scale: float):
    """Whole fixed-order decode step for one KV head.  ``index`` is a dict with coarse, codebooks,
    codes, list_ids, norms, vbar over the n indexed keys.  Returns (out, topk_idx, logits)."""
    length = keys.shape[0]
    sink_end = min(sink, length)
    n = index["codes"].shape[0]
    assert n == max(sink_end, length - local) - sink_end or local == 0
    qnorm, lut, list_scores = lut_build(queries, index["coarse"], index["codebooks"])
    logits = scan(index["codes"], index["list_ids"], index["norms"], lut, list_scores, qnorm, scale)
    k = resolve_topk(n, fraction)
    idx, _ = topk(logits, k)
    out = attend(queries, keys, values, sink_end, logits, idx, index["list_ids"], index["vbar"], scale)
    return out, idx, logits
