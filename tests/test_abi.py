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

    index.n_cap = 1 << 18
    assert launches(4, 16384) == 1
    assert launches(4, 16385) == 4            # more keys than a workgroup holds in registers
    assert launches(4, 8192, appending=1) == 4
    assert launches(16, 8192) == 1 and launches(16, 8192) == launches(16, 1)
    index.batch = 3                           # 3 * 8 * 16 query rows > 256: two rows per workgroup
    assert launches(16, 8192) == 4
    index.batch = 5                           # 5 * 8 * 16 / 2 workgroups > 256
    assert launches(16, 8192) == 5
    index.batch = 1
    sel.flags = _lib.SELECT_GENERAL_PATH
    assert launches(4, 8192) == 4
    sel.flags, sel.k_cap = 0, 2049
    assert launches(4, 8192) == 4
    # tables and threshold estimate in one launch: unless the caller keeps them apart, for steps
    # whose query rows, or pairs of them (streams padded to a multiple of 8; one more workgroup per
    # stream in a step that appends), each get a compute unit, with at most 512 lists and 8 192
    # sampled keys per stream
    sel.flags = _lib.SELECT_SEPARATE_TABLES
    assert launches(4, 8192) == 5
    sel.flags = 0
    index.batch = 9                           # 72 streams x 4 rows > 256: two rows per workgroup
    assert launches(4, 20000) == 4
    index.batch = 16                          # 128 streams x 2 pairs = 256
    assert launches(4, 20000) == 4 and launches(4, 20000, appending=1) == 5   # (one more workgroup per stream)
    index.batch = 17
    assert launches(4, 20000) == 5
    index.batch = 7                           # 56 streams x 4 rows; with the appending workgroups 224 + 56: pairs
    assert launches(4, 20000) == 4 and launches(4, 20000, appending=1) == 4
    index.batch, index.kv_heads = 7, 9        # 63 streams, padded to 64: 256 rows, or 256 pairs of a group of 5 (padded to 8)
    assert launches(4, 20000) == 4 and launches(5, 20000) == 4 and launches(9, 20000) == 5
    index.batch, index.kv_heads = 1, 8
    index.num_lists = 513
    assert launches(4, 20000) == 5
    index.num_lists, index.s_cap = 512, 8200
    assert launches(4, 20000) == 5
    index.s_cap = 8192
    assert launches(4, 20000) == 4
    # scan + selection + attention in one launch: only when asked for, and only for shapes it serves
    sel.flags = _lib.SELECT_ONE_LAUNCH
    assert launches(4, 20000) == 3 and launches(7, 20000) == 3
    assert launches(4, 8192) == 3 and launches(2, 20000) == 4 and launches(16, 20000) == 4
    sel.k_cap = 328
    assert launches(4, 8192) == 1             # (the short-context kernel comes first)
    index.batch, sel.n_mean = 4, 0            # several sequences of unknown lengths
    assert launches(4, 20000) == 4
    sel.n_mean = 19000                        # ... of about one length
    assert launches(4, 20000) == 3
    sel.n_mean = 9000
    assert launches(4, 20000) == 4
    index.n_cap = (1 << 20) + 8               # stored positions no longer fit a candidate record's 20 bits
    index.batch, sel.n_mean = 1, 0
    assert launches(4, 20000) == 4


def test_short_context_rule_counts_the_whole_lds_footprint():
    import ctypes

    lib = _lib.load()
    index, sel = _lib.Index(), _lib.Select()
    index.batch, index.kv_heads = 1, 8

    def launches(lists, k_cap):
        index.num_lists, sel.k_cap = lists, k_cap
        return lib.pqhsa_decode_step_launches(ctypes.byref(index), 4, 8192, ctypes.byref(sel), 0)

    assert launches(512, 2048) == 1
    assert launches(1024, 512) == 1
    # 135 168 + 8 L + 4 k_cap bytes of dynamic LDS plus the static arrays pass 160 KB at this corner
    assert launches(1024, 2048) != 1


def header_struct_fields(name):
    text = open(os.path.join(ROOT, "include", "pqhsa.h")).read()
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    return [re.search(r"(\w+)\s*$", decl.strip()).group(1) for decl in body.split(";") if decl.strip()]


def test_ctypes_mirrors_follow_the_header_field_order():
    for cname, mirror in (("pqhsa_kv_view", _lib.KvView), ("pqhsa_select", _lib.Select), ("pqhsa_index", _lib.Index)):
        assert [f[0] for f in mirror._fields_] == header_struct_fields(cname), cname


def test_integration_document_stub_matches_the_library_structs():
    """The ctypes binding that the integration notes at the repository root show is built from their
    text and laid over the library's mirrors: same fields, same offsets, same sizes, and the argument
    list of pqhsa_decode_step."""
    import ctypes

    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r"```python\n(import ctypes, torch.*?)```", text, flags=re.S).group(1)
    structs = block[block.index("c_void_p, c_int32"):block.index("# pqhsa_index")]
    ns = {"ctypes": ctypes}
    exec(structs, ns)  # two ctypes.Structure definitions written in this repository's own document
    for doc, mirror in ((ns["KvView"], _lib.KvView), (ns["Select"], _lib.Select)):
        assert ctypes.sizeof(doc) == ctypes.sizeof(mirror)
        assert [f[0] for f in doc._fields_] == [f[0] for f in mirror._fields_]
        for fname, _ in mirror._fields_:
            assert getattr(doc, fname).offset == getattr(mirror, fname).offset, fname
            assert getattr(doc, fname).size == getattr(mirror, fname).size, fname
    argtypes = re.search(r"pqhsa_decode_step\.argtypes = \[(.*?)\]", block, flags=re.S).group(1)
    argtypes = re.sub(r"#[^\n]*", "", argtypes)
    names = [a.strip() for a in argtypes.replace("\n", " ").split(",") if a.strip()]
    ns.update(P=ctypes.POINTER, Index=_lib.Index)
    got = [eval(a, ns) for a in names]
    want = _lib.SIGNATURES["pqhsa_decode_step"][1]
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert ctypes.sizeof(g) == ctypes.sizeof(w)
        assert (g is w) or (hasattr(g, "_type_") and hasattr(w, "_type_") and
                            [f[0] for f in getattr(g._type_, "_fields_", [])] == [f[0] for f in getattr(w._type_, "_fields_", [])])


def test_stand_alone_scan_statistics_reject_bad_arguments_before_any_gpu_work():
    """pqhsa_lut_scan_stats and pqhsa_block_reduce check their arguments before the first HIP call:
    the error code and message come back on a machine without a GPU too."""
    import ctypes

    lib = _lib.load()
    idx = _lib.Index()
    idx.batch, idx.kv_heads, idx.num_lists, idx.n_cap = 1, 1, 16, 1024
    p = 4096  # stands for device pointers that a rejected call never follows

    def stats(G=4, n_max=1000, block_keys=512, blocks=2, qnorm=p):
        return lib.pqhsa_lut_scan_stats(ctypes.byref(idx), G, n_max, qnorm, p, p, 1.0, block_keys, blocks, p, p, None)

    assert stats(qnorm=None) == -1 and b"NULL" in lib.pqhsa_last_error()
    assert stats(G=17) == -1 and b"G=17" in lib.pqhsa_last_error()
    assert stats(n_max=2000) == -1 and b"n_max=2000" in lib.pqhsa_last_error()
    assert stats(blocks=1) == -1 and b"do not cover" in lib.pqhsa_last_error()
    assert stats(block_keys=0) == -1
    idx.num_lists = 4096                     # 4096 lists x 16 padded rows of list scores: more than a compute unit's LDS
    assert stats(G=16) == -1 and b"LDS" in lib.pqhsa_last_error()
    assert lib.pqhsa_block_reduce(None, p, 4, 8, p, p, None) == -1 and b"NULL" in lib.pqhsa_last_error()
    assert lib.pqhsa_block_reduce(p, p, 4, 0, p, p, None) == -1 and b"blocks=0" in lib.pqhsa_last_error()
    assert lib.pqhsa_block_reduce(p, p, 0, 8, p, p, None) == 0          # no rows: nothing to do
