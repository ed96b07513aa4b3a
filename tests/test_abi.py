"""The C-ABI library loads without a GPU and exports every symbol ``include/pqhsa.h`` declares."""

import os
import re

from pqhsa_release_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "pqhsa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pqhsa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/pqhsa.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)


def test_version_and_helpers_run_without_a_gpu():
    lib = _lib.load()
    assert b"gfx950" in lib.pqhsa_version()
    assert [lib.pqhsa_padded_groups(g) for g in (1, 2, 3, 4, 5, 7, 8, 9, 16)] == [1, 2, 4, 4, 8, 8, 8, 16, 16]
    assert lib.pqhsa_decode_workspace_bytes(1, 8, 4, 32704, 512, 654) > 0
    assert lib.pqhsa_topk_workspace_bytes(4, 1000) > 0
    assert lib.pqhsa_attend_workspace_bytes(1, 8, 4, 512) > 0


def test_struct_layouts_match_the_header():
    import ctypes

    # sizes implied by include/pqhsa.h on LP64: pointers and int64 8-byte aligned
    assert ctypes.sizeof(_lib.KvView) == 8 + 8 + 4 + 4 + 8 * 4 + 4 + 4 + 8
    assert ctypes.sizeof(_lib.Index) == 15 * 8 + 2 * 8 + 4 * 3 + 4
    assert ctypes.sizeof(_lib.Select) == 24


def test_launch_count_follows_the_short_context_rule():
    import ctypes

    lib = _lib.load()
    index, sel = _lib.Index(), _lib.Select()
    index.batch, index.kv_heads, index.num_lists = 1, 8, 512
    sel.k_cap = 328

    def launches(groups, n_max, appending=0):
        return lib.pqhsa_decode_step_launches(ctypes.byref(index), groups, n_max, ctypes.byref(sel), appending)

    assert launches(4, 16384) == 1
    assert launches(4, 16385) == 5            # more keys than a workgroup holds in registers
    assert launches(4, 8192, appending=1) == 5
    assert launches(16, 8192) == 1 and launches(16, 8192) == launches(16, 1)
    index.batch = 3                           # 3 * 8 * 16 query rows > 256
    assert launches(16, 8192) == 5
    index.batch = 1
    sel.flags = _lib.SELECT_GENERAL_PATH
    assert launches(4, 8192) == 5
    sel.flags, sel.k_cap = 0, 2049
    assert launches(4, 8192) == 5
