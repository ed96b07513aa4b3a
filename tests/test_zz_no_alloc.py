"""pqhsa_decode_step_static (the entry point that allocates nothing: its scratch is a device array
built into the library) gives the results of pqhsa_decode_step, on two calls in a row that share
the array, the second on a smaller input."""

import ctypes

import numpy as np
import pytest
import torch

from pqhsa_release_amd import _lib, ops
from tests.gpu_util import SCALE, Problem

pytestmark = pytest.mark.gpu


def _both_ways(p, fraction):
    lib = _lib.load()
    idx = p.device_index("cuda")
    kv = ops.kv_paged(*p.paged_kv("5d"))
    k_cap = max(ops.resolve_topk(p.n_max, fraction, 0), 1)
    rows = p.B * p.H * p.G
    q = p.q_tensor().float()
    seq_lens = p.seq_lens()
    # the existing entry point, with a caller workspace
    ws = ops.DecodeWorkspace(idx, p.G, k_cap)
    want_out = torch.full_like(q, float("nan"))  # a row no workgroup folds would stay NaN
    ops.decode_step(q, want_out, kv, idx, p.G, seq_lens, sink=p.sink, full_max=p.sink + p.local, fraction=fraction,
                    topk=0, scale=SCALE, workspace=ws)
    torch.cuda.synchronize()
    # the static-scratch entry point, straight through the C ABI: inputs and outputs only
    assert ws.bytes <= lib.pqhsa_static_scratch_bytes()
    out = torch.full_like(q, float("nan"))
    tidx = torch.full((rows, k_cap), -1, dtype=torch.int32, device="cuda")
    tval = torch.zeros(rows, k_cap, dtype=torch.float32, device="cuda")
    tcnt = torch.zeros(rows, dtype=torch.int32, device="cuda")
    sel = _lib.Select()
    sel.fraction, sel.topk, sel.k_cap = float(fraction), 0, k_cap
    rc = lib.pqhsa_decode_step_static(q.data_ptr(), _lib.F32, out.data_ptr(), kv.ref(), idx.ref(), p.G,
                                      seq_lens.data_ptr(), p.sink, idx.n_max, p.sink + p.local, ctypes.byref(sel),
                                      SCALE, ops.EPS, tidx.data_ptr(), tval.data_ptr(), tcnt.data_ptr(),
                                      torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "pqhsa_decode_step_static")
    torch.cuda.synchronize()
    cnt = tcnt.cpu().numpy()
    assert np.array_equal(cnt, ws.topk_cnt.cpu().numpy())
    got_i, want_i = tidx.cpu().numpy(), ws.topk_idx.cpu().numpy()
    got_v, want_v = tval.cpu().numpy(), ws.topk_val.cpu().numpy()
    for r in range(rows):  # the same keys with the same logits, bit for bit (their order is free)
        k = int(cnt[r])
        go, wo = np.argsort(got_i[r, :k], kind="stable"), np.argsort(want_i[r, :k], kind="stable")
        assert np.array_equal(got_i[r, :k][go], want_i[r, :k][wo]), r
        assert np.array_equal(got_v[r, :k][go], want_v[r, :k][wo]), r
    # the per-list sums are float atomics in both entry points: equal up to their summation order
    err = float((out - want_out).abs().max())
    assert err <= 2e-5, err
    return err


def test_static_scratch_entry_point_matches_the_workspace_one_twice_in_a_row():
    big = Problem(lens=[5200, 3100], heads=2, groups=4, lists=64, dtype=torch.bfloat16, seed=71)
    small = Problem(lens=[900], heads=1, groups=3, lists=16, dtype=torch.bfloat16, seed=72)
    e1 = _both_ways(big, 0.02)
    e2 = _both_ways(small, 0.05)   # shares the array with the call before it, which left its contents there
    print(f"static scratch vs workspace: max abs output difference {e1:.2e}, {e2:.2e}")


def test_static_scratch_entry_point_rejects_a_shape_beyond_its_array():
    lib = _lib.load()
    idx = ops.DeviceIndex(16, 8, 512, 1 << 17, "cuda")   # 512 query rows x 20 000 selected keys: far more scratch
    need = lib.pqhsa_decode_workspace_bytes(16, 8, 4, idx.n_cap, 512, 20000)
    assert need > lib.pqhsa_static_scratch_bytes()
    sel = _lib.Select()
    sel.fraction, sel.topk, sel.k_cap = 0.0, 20000, 20000
    kvt = torch.zeros(2, 4, 16, 8, 128, dtype=torch.bfloat16, device="cuda")
    table = torch.zeros(16, 2, dtype=torch.int32, device="cuda")
    kv = ops.kv_paged(kvt, table)
    q = torch.zeros(16, 32, 128, device="cuda")
    sl = torch.zeros(16, dtype=torch.int32, device="cuda")
    rc = lib.pqhsa_decode_step_static(q.data_ptr(), _lib.F32, q.data_ptr(), kv.ref(), idx.ref(), 4, sl.data_ptr(), 4, 0,
                                      68, ctypes.byref(sel), SCALE, ops.EPS, None, None, None,
                                      torch.cuda.current_stream().cuda_stream)
    assert rc == -3
    assert b"scratch" in lib.pqhsa_last_error()
