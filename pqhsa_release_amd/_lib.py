"""ctypes binding of ``libpqhsa.so`` (the C ABI declared in ``include/pqhsa.h``).

There is no CPU fallback: if the shared library is missing, or a call fails, an exception is
raised.
"""

from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libpqhsa.so")

F32, BF16, F16 = 0, 1, 2

c_void_p = ctypes.c_void_p
c_int32 = ctypes.c_int32
c_int64 = ctypes.c_int64
c_float = ctypes.c_float
c_size_t = ctypes.c_size_t


class KvView(ctypes.Structure):
    _fields_ = [
        ("k_base", c_void_p),
        ("v_base", c_void_p),
        ("dtype", c_int32),
        ("paged", c_int32),
        ("stride_seq", c_int64),
        ("stride_head", c_int64),
        ("stride_tok", c_int64),
        ("stride_block", c_int64),
        ("block_size", c_int32),
        ("max_blocks", c_int32),
        ("block_table", c_void_p),
    ]


class Index(ctypes.Structure):
    _fields_ = [
        ("codes", c_void_p),
        ("list_ids", c_void_p),
        ("norms", c_void_p),
        ("pos", c_void_p),
        ("coarse", c_void_p),
        ("codebooks", c_void_p),
        ("vbar", c_void_p),
        ("vsum", c_void_p),
        ("vcount", c_void_p),
        ("n_idx", c_void_p),
        ("n_sorted", c_void_p),
        ("s_codes", c_void_p),
        ("s_list_ids", c_void_p),
        ("s_norms", c_void_p),
        ("s_n", c_void_p),
        ("s_cap", c_int64),
        ("n_cap", c_int64),
        ("num_lists", c_int32),
        ("batch", c_int32),
        ("kv_heads", c_int32),
    ]


class Select(ctypes.Structure):
    _fields_ = [("fraction", ctypes.c_double), ("topk", c_int32), ("k_cap", c_int32), ("flags", c_int32),
                ("n_mean", c_int32)]


SELECT_GENERAL_PATH = 1
SELECT_ONE_LAUNCH = 2
SELECT_SHARE_ROWS = 4
SELECT_SEPARATE_TABLES = 8


class PqhsaError(RuntimeError):
    pass


_P = ctypes.POINTER

# name -> (restype, argtypes); every symbol declared in include/pqhsa.h
SIGNATURES = {
    "pqhsa_version": (ctypes.c_char_p, []),
    "pqhsa_last_error": (ctypes.c_char_p, []),
    "pqhsa_padded_groups": (c_int32, [c_int32]),
    "pqhsa_encode": (ctypes.c_int, [_P(KvView), _P(Index), c_int32, c_void_p, c_void_p, c_int32, c_float, c_void_p]),
    "pqhsa_encode_bulk_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "pqhsa_encode_bulk": (ctypes.c_int, [_P(KvView), _P(Index), c_int32, c_void_p, c_void_p, c_int32, c_float,
                                         c_void_p, c_size_t, c_void_p]),
    "pqhsa_nearest_rows_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32]),
    "pqhsa_nearest_rows": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_float, c_void_p, c_int64,
                                          c_void_p, c_size_t, c_void_p]),
    "pqhsa_nearest_codewords": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int64, c_void_p, c_int64, c_void_p]),
    "pqhsa_nearest_from_products": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_int64,
                                                   c_void_p]),
    "pqhsa_value_summaries": (ctypes.c_int, [_P(KvView), _P(Index), c_int32, c_int32, c_void_p]),
    "pqhsa_encode_append": (ctypes.c_int, [_P(KvView), _P(Index), c_int32, c_void_p, c_void_p, c_int32, c_float,
                                           c_void_p]),
    "pqhsa_lut_build": (ctypes.c_int, [c_void_p, c_int32, _P(Index), c_int32, c_float, c_void_p, c_void_p, c_void_p,
                                       c_void_p]),
    "pqhsa_lut_scan": (ctypes.c_int, [_P(Index), c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_float, c_void_p,
                                      c_int64, c_void_p]),
    "pqhsa_topk_workspace_bytes": (c_size_t, [c_int32, c_int64]),
    "pqhsa_topk_radix": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                        c_int32, c_void_p, c_size_t, c_void_p]),
    "pqhsa_decode_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int64, c_int32, c_int32]),
    "pqhsa_decode_step": (ctypes.c_int, [c_void_p, c_int32, c_void_p, _P(KvView), _P(Index), c_int32, c_void_p,
                                         c_int32, c_int32, c_int32, _P(Select), c_float, c_float, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_size_t, c_void_p]),
    "pqhsa_static_scratch_bytes": (c_size_t, []),
    "pqhsa_decode_step_static": (ctypes.c_int, [c_void_p, c_int32, c_void_p, _P(KvView), _P(Index), c_int32, c_void_p,
                                                c_int32, c_int32, c_int32, _P(Select), c_float, c_float, c_void_p,
                                                c_void_p, c_void_p, c_void_p]),
    "pqhsa_append_decode_step": (ctypes.c_int, [c_void_p, c_int32, c_void_p, _P(KvView), _P(Index), c_int32, c_void_p,
                                                c_int32, c_int32, c_int32, _P(Select), c_float, c_float, c_void_p,
                                                c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "pqhsa_decode_rescan_counter": (c_void_p, [c_void_p]),
    "pqhsa_decode_candidate_counts": (c_void_p, [c_void_p]),
    "pqhsa_decode_fused_aborts": (c_void_p, [c_void_p]),
    "pqhsa_attend_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "pqhsa_hybrid_attend_paged": (ctypes.c_int, [c_void_p, c_int32, c_void_p, _P(KvView), _P(Index), c_int32,
                                                 c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int32,
                                                 c_void_p, c_int64, c_void_p, c_void_p, c_float, c_void_p, c_size_t,
                                                 c_void_p]),
    "pqhsa_paged_gather_range": (ctypes.c_int, [_P(KvView), c_int32, c_int32, c_int64, c_int64, c_void_p, c_void_p,
                                                c_void_p]),
    "pqhsa_profile_enable": (ctypes.c_int, [c_int32]),
    "pqhsa_profile_only": (ctypes.c_int, [c_int32]),
    "pqhsa_profile_every": (ctypes.c_int, [c_int32]),
    "pqhsa_profile_collect": (ctypes.c_int, [c_void_p, c_void_p]),
    "pqhsa_paged_gather_at": (ctypes.c_int, [_P(KvView), c_int32, c_int32, c_void_p, c_int64, c_void_p, c_void_p,
                                             c_void_p]),
    "pqhsa_lut_scan_mass": (ctypes.c_int, [_P(Index), c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_float, c_void_p,
                                           c_void_p, c_void_p]),
    "pqhsa_lut_scan_stats": (ctypes.c_int, [_P(Index), c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_float, c_int32,
                                            c_int32, c_void_p, c_void_p, c_void_p]),
    "pqhsa_block_reduce": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p]),
    "pqhsa_decode_step_launches": (c_int32, [_P(Index), c_int32, c_int32, _P(Select), c_int32]),
    "pqhsa_gather_probe": (ctypes.c_int, [_P(KvView), c_int32, c_int32, c_void_p, c_int64, c_void_p, c_void_p]),
}

_LIB: ctypes.CDLL | None = None


def load() -> ctypes.CDLL:
    """Load the shared library (once) and attach the signatures."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = os.environ.get("PQHSA_LIBRARY", LIB_PATH)  # another build of the same ABI, e.g. a tuning build
    if not os.path.exists(path):
        raise PqhsaError(
            f"{path} is missing: build it with `python -m pqhsa_release_amd.build` "
            "(hipcc, gfx950); there is no fallback path"
        )
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().pqhsa_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(f"{what}: {msg}")
        raise PqhsaError(f"{what} failed ({rc}): {msg}")
