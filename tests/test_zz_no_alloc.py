"""kge_rank_filtered_static (the entry point that allocates nothing) against kge_rank_filtered, through the C ABI.

Two calls in a row on one GPU, the second with a smaller input: the static scratch array keeps what the first call
left in it, and nothing of that may reach the second call's results.  Collected last on purpose: a failure here
must not hide the other GPU tests.
"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import random_tables, random_hr, stored_tables, dev, random_csr

pytestmark = pytest.mark.gpu


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _both(lib, Q, bias, E, dtype, scale, target, rows, row_ptr, col):
    """(outputs of kge_rank_filtered, outputs of kge_rank_filtered_static) for the same arguments."""
    B, d = Q.shape
    N = E.shape[0]
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n_rows = 0 if row_ptr is None else row_ptr.numel() - 1

    def outputs():
        return ([torch.full((B,), -77, dtype=torch.int32, device="cuda") for _ in range(3)]
                + [torch.full((B,), float("nan"), dtype=torch.float32, device="cuda")])

    want = outputs()
    ws_bytes = lib.kge_rank_workspace_bytes(B)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device="cuda")
    rc = lib.kge_rank_filtered(_p(Q), _p(bias), _p(E), dtype, _p(scale), B, d, N, _p(target), _p(rows), _p(row_ptr),
                               _p(col), n_rows, _p(want[0]), _p(want[1]), _p(want[2]), _p(want[3]), _p(ws), ws_bytes, st)
    assert rc == 0, lib.kge_last_error()
    got = outputs()
    assert lib.kge_rank_static_init() == 0, lib.kge_last_error()
    torch.cuda.synchronize()
    held, free = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.kge_rank_filtered_static(_p(Q), _p(bias), _p(E), dtype, _p(scale), B, d, N, _p(target), _p(rows),
                                      _p(row_ptr), _p(col), n_rows, _p(got[0]), _p(got[1]), _p(got[2]), _p(got[3]), st)
    assert rc == 0, lib.kge_last_error()
    torch.cuda.synchronize()
    # the call allocated nothing: neither through torch's allocator nor behind its back
    assert torch.cuda.memory_allocated() == held and torch.cuda.mem_get_info()[0] == free
    return want, got


@pytest.mark.parametrize("storage,d", [("bf16", 128), ("fp32", 40), ("int8", 64)])
def test_rank_filtered_static_equals_rank_filtered_on_two_calls_in_a_row(storage, d):
    from dicee_amd import _lib, ops
    from dicee_amd.csr import FilterCSR
    lib = _lib.load()
    dtype = {"fp32": _lib.DTYPE_F32, "bf16": _lib.DTYPE_BF16, "int8": _lib.DTYPE_I8}[storage]
    rng = np.random.default_rng(31)
    N, R = 7000, 5
    E, Rel = random_tables(rng, N, R, d)
    Et, sc, Rt, _, _ = stored_tables(E, Rel, storage)
    Eg, scg = dev(Et), dev(sc)
    # first call: 9000 queries (two sub-batches of the filter correction, hub rows, shared rows);
    # second call: 700 queries with other filters: everything the first call left in the scratch is stale
    for B, n_pairs, hubs in ((9000, 60, [(0, 4000), (5, 1500)]), (700, 500, [(3, 900)])):
        hr = random_hr(rng, n_pairs, R, B)
        targets = rng.integers(0, N, B).astype(np.int64)
        er = random_csr(rng, hr, targets, N, R, max_len=5, hub_rows=hubs)
        csr = FilterCSR.from_er_vocab(er, R, device="cuda")
        hr_g = dev(torch.from_numpy(hr))
        Q, bias = ops.build_query("DistMult", Eg, dev(Rt), hr_g, ent_scale=scg)
        bias = bias + 0.25
        rows = csr.rows_for(hr_g)
        tg = dev(torch.from_numpy(targets))
        want, got = _both(lib, Q, bias, Eg, dtype, scg, tg, rows, csr.row_ptr, csr.col)
        for w, g, name in zip(want, got, ("n_greater", "n_equal", "n_equal_lower", "target_score")):
            assert torch.equal(w, g), (name, B)
        assert int(want[0].min()) >= 0 and int((want[0] >= 0).sum()) == B
        # without a filter
        want, got = _both(lib, Q, None, Eg, dtype, scg, tg, None, None, None)
        for w, g in zip(want, got):
            assert torch.equal(w, g)


def test_rank_filtered_static_rejects_what_does_not_fit():
    from dicee_amd import _lib
    lib = _lib.load()
    B = 65536 + 1
    Q = torch.zeros((B, 16), device="cuda")
    E = torch.zeros((100, 16), device="cuda")
    t = torch.zeros((B,), dtype=torch.int64, device="cuda")
    o = [torch.zeros((B,), dtype=torch.int32, device="cuda") for _ in range(3)]
    ts = torch.zeros((B,), dtype=torch.float32, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.kge_rank_filtered_static(_p(Q), None, _p(E), _lib.DTYPE_F32, None, B, 16, 100, _p(t), None, None, None, 0,
                                      _p(o[0]), _p(o[1]), _p(o[2]), _p(ts), st)
    assert rc == 3                                                    # KGE_ERR_WORKSPACE
    assert b"exceeds" in lib.kge_last_error() and b"65536" in lib.kge_last_error()
    # the largest batch that fits runs
    B = 65536
    rc = lib.kge_rank_filtered_static(_p(Q[:B]), None, _p(E), _lib.DTYPE_F32, None, B, 16, 100, _p(t[:B]), None, None,
                                      None, 0, _p(o[0]), _p(o[1]), _p(o[2]), _p(ts), st)
    assert rc == 0, lib.kge_last_error()
    torch.cuda.synchronize()
    assert int(o[1][:B].min()) == 99 and int(o[0][:B].max()) == 0     # all-zero scores: every other entity ties
