"""Parity of the HIP kernels (through the C ABI) against the CPU oracle on seeded inputs.

Bars: fp32 scores within 1e-5 relative, bf16 / int8 within 2e-2 relative (relative to
max(|s|, row RMS)); ranks, tie counters and top-k indices bit-exact with respect to the scores the
library itself materialises, and inside the oracle's tolerance interval.
"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import RTOL, score_close, random_tables, random_hr, stored_tables, dev, random_csr
from oracle import kge_oracle as ko

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from dicee_amd import ops as _ops
    return _ops


@pytest.fixture(scope="module")
def FilterCSR():
    from dicee_amd.csr import FilterCSR as F
    return F


MODEL_CASES = [
    # model, d, kwargs
    ("DistMult", 32, {}),
    ("ComplEx", 200, {}),
    ("QMult", 128, {}),
    ("QMult", 64, {"normalize_relation": False}),
    ("Keci", 256, {"p": 0, "q": 1, "coeff_q": [1.0]}),
    ("Keci", 28, {"p": 1, "q": 2, "coeff_p": [0.7], "coeff_q": [1.3, -0.4]}),
    ("Keci", 35, {"p": 3, "q": 3, "coeff_p": [0.7, 1.1, -0.3], "coeff_q": [1.3, -0.4, 0.9]}),
    ("Keci", 24, {"p": 2, "q": 0, "coeff_p": [0.5, 2.0]}),
    ("Keci", 16, {"p": 0, "q": 0}),
    ("OMult", 128, {}),
    ("OMult", 24, {"normalize_relation": False}),
    ("DeCaL", 28, {"p": 2, "q": 2, "r": 2, "coeff_p": [0.7, 1.1], "coeff_q": [1.3, -0.4], "coeff_r": [0.6, 1.2]}),
    ("DeCaL", 256, {"p": 3, "q": 1, "r": 3, "coeff_p": [0.7, 1.1, -0.3], "coeff_q": [1.3], "coeff_r": [0.6, 1.2, -0.9]}),
    ("DeCaL", 24, {"p": 0, "q": 0, "r": 2, "coeff_r": [0.5, 2.0]}),
    ("DeCaL", 20, {"p": 1, "q": 1, "r": 2, "coeff_p": [0.7], "coeff_q": [1.3], "coeff_r": [0.6, 1.2]}),
    ("DeCaL", 18, {"p": 1, "q": 1, "r": 0, "coeff_p": [0.7], "coeff_q": [1.3]}),
]


def _gpu_kwargs(kw):
    out = dict(kw)
    for k in ("coeff_p", "coeff_q", "coeff_r"):
        if k in out:
            out[k] = torch.tensor(out[k], dtype=torch.float32, device="cuda")
    return out


@pytest.mark.parametrize("model,d,kw", MODEL_CASES)
def test_build_query_fp32(ops, model, d, kw):
    rng = np.random.default_rng(100 + d)
    N, R, B = 300, 17, 77
    E, Rel = random_tables(rng, N, R, d, std=0.5)
    hr = random_hr(rng, N, R, B)
    Q, bias = ops.build_query(model, dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)),
                              dev(torch.from_numpy(hr)), **_gpu_kwargs(kw))
    Qr, br = ko.build_query(model, E, Rel, hr, **kw)
    ok, worst = score_close(Q.cpu().numpy(), Qr, 1e-5)
    assert ok, worst
    ok, worst = score_close(bias.cpu().numpy(), br, 1e-5)
    assert ok or np.abs(br).max() == 0, worst
    if np.abs(br).max() == 0:
        assert float(bias.abs().max()) == 0.0


@pytest.mark.parametrize("storage", ["bf16", "int8"])
@pytest.mark.parametrize("model", ["DistMult", "ComplEx", "QMult", "OMult"])
def test_build_query_quantised_tables(ops, model, storage):
    rng = np.random.default_rng(7)
    N, R, d, B = 200, 9, 128, 50
    E, Rel = random_tables(rng, N, R, d)
    hr = random_hr(rng, N, R, B)
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Q, _ = ops.build_query(model, dev(Et), dev(Rt), dev(torch.from_numpy(hr)), ent_scale=dev(sc))
    Qr, _ = ko.build_query(model, Ev, Rv, hr)
    ok, worst = score_close(Q.cpu().numpy(), Qr, 1e-5)      # the gather itself is exact fp32 math
    assert ok, worst


@pytest.mark.parametrize("kind", ["LayerNorm", "BatchNorm1d"])
def test_build_query_with_normalisation(ops, kind):
    rng = np.random.default_rng(8)
    N, R, d, B = 100, 5, 48, 40
    E, Rel = random_tables(rng, N, R, d, std=1.0)
    hr = random_hr(rng, N, R, B)
    a_h, a_r = rng.normal(size=d).astype(np.float32), rng.normal(size=d).astype(np.float32)
    b_h, b_r = rng.uniform(0.5, 2, d).astype(np.float32), rng.uniform(0.5, 2, d).astype(np.float32)
    if kind == "LayerNorm":
        onorm = {"kind": kind, "h_weight": a_h, "h_bias": b_h, "r_weight": a_r, "r_bias": b_r}
    else:
        onorm = {"kind": kind, "h_mean": a_h, "h_var": b_h, "r_mean": a_r, "r_var": b_r}
    gnorm = {"kind": kind, "eps": 1e-5, "h_a": dev(torch.from_numpy(a_h)), "h_b": dev(torch.from_numpy(b_h)),
             "r_a": dev(torch.from_numpy(a_r)), "r_b": dev(torch.from_numpy(b_r))}
    for model in ("ComplEx", "QMult"):
        kw = {"normalize_relation": False} if model == "QMult" else {}
        Q, _ = ops.build_query(model, dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)),
                               dev(torch.from_numpy(hr)), norm=gnorm, **kw)
        Qr, _ = ko.build_query(model, E, Rel, hr, norm=onorm, **kw)
        ok, worst = score_close(Q.cpu().numpy(), Qr, 2e-5)
        assert ok, worst


def test_build_query_bad_ids_give_nan_not_fault(ops):
    rng = np.random.default_rng(9)
    E, Rel = random_tables(rng, 50, 4, 16)
    hr = np.array([[0, 0], [50, 1], [3, 4], [-1, 0], [49, 3]], dtype=np.int64)
    Q, bias = ops.build_query("DistMult", dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)),
                              dev(torch.from_numpy(hr)))
    Q = Q.cpu().numpy()
    assert np.isnan(Q[1]).all() and np.isnan(Q[2]).all() and np.isnan(Q[3]).all()
    assert np.isfinite(Q[0]).all() and np.isfinite(Q[4]).all()


SCORE_CASES = [
    # model, N, R, d, B, storage, kw
    ("DistMult", 135, 46, 32, 512, "fp32", {}),
    ("ComplEx", 1003, 11, 200, 301, "fp32", {}),
    ("Keci", 257, 6, 28, 33, "fp32", {"p": 1, "q": 2, "coeff_p": [0.7], "coeff_q": [1.3, -0.4]}),
    ("Keci", 300, 6, 35, 70, "fp32", {"p": 3, "q": 3, "coeff_p": [0.7, 1.1, -0.3], "coeff_q": [1.3, -0.4, 0.9]}),
    ("DistMult", 64, 3, 7, 5, "fp32", {}),
    ("QMult", 999, 5, 128, 130, "bf16", {}),
    ("DistMult", 5000, 7, 128, 600, "bf16", {}),
    ("ComplEx", 321, 7, 64, 40, "bf16", {}),
    ("Keci", 1500, 6, 256, 300, "bf16", {"p": 0, "q": 1, "coeff_q": [1.0]}),      # d = 256: the streaming kernel, 512-byte rows
    ("DistMult", 9001, 5, 256, 700, "bf16", {}),     # the same over several stages per workgroup, partial last groups
    ("DistMult", 500, 5, 384, 90, "bf16", {}),       # wider still: the query row in registers, rows through LDS by segments
    ("DistMult", 9001, 5, 512, 700, "bf16", {}),     # the widest of that kernel, several stages and chunks, partial last groups
    ("ComplEx", 4100, 5, 400, 300, "bf16", {}),      # its four-segment form on rows whose LDS tail stays zero
    ("DistMult", 4100, 5, 264, 300, "bf16", {}),     # its three-segment form likewise
    ("DistMult", 600, 5, 520, 90, "bf16", {}),       # wider than any register-resident form: kchunk_kernel
    ("ComplEx", 700, 7, 200, 150, "bf16", {}),       # between 128 and 256: the d = 256 kernels on rows whose LDS tail stays zero
    ("DistMult", 300, 5, 136, 70, "bf16", {}),
    ("ComplEx", 9001, 5, 200, 700, "bf16", {}),      # the same over several stages per workgroup, partial last groups
    ("DistMult", 777, 9, 128, 70, "int8", {}),
    ("ComplEx", 2100, 9, 96, 520, "int8", {}),
    ("ComplEx", 1300, 7, 256, 300, "int8", {}),      # int8 d = 256: one query tile per wave
    ("DistMult", 777, 5, 144, 131, "int8", {}),      # between 128 and 256: the same kernel, rows padded with zeros in LDS
    ("DistMult", 9001, 5, 240, 700, "int8", {}),
    ("DistMult", 400, 5, 272, 90, "int8", {}),       # wider than 256: widened to bf16 on the way into the segmented LDS rows
    ("DistMult", 9001, 5, 512, 700, "int8", {}),
    ("ComplEx", 4100, 5, 400, 300, "int8", {}),
    ("DistMult", 600, 5, 528, 90, "int8", {}),       # wider than any register-resident form: kchunk_kernel, scales applied per tile
]


def _setup(ops, model, N, R, d, B, storage, kw, seed=0, std=0.1):
    rng = np.random.default_rng(seed)
    E, Rel = random_tables(rng, N, R, d, std=std)
    hr = random_hr(rng, N, R, B)
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Eg, scg = dev(Et), dev(sc)
    Q, bias = ops.build_query(model, Eg, dev(Rt), dev(torch.from_numpy(hr)), ent_scale=scg, **_gpu_kwargs(kw))
    return rng, hr, Eg, scg, Q, bias, Ev, Rv


@pytest.mark.parametrize("model,N,R,d,B,storage,kw", SCORE_CASES)
def test_scores_vs_oracle(ops, model, N, R, d, B, storage, kw):
    rng, hr, Eg, scg, Q, bias, Ev, Rv = _setup(ops, model, N, R, d, B, storage, kw)
    S = ops.scores(Q, bias, Eg, scg).cpu().numpy()
    ref = ko.k_vs_all_scores(model, Ev, Rv, hr, **kw)
    ok, worst = score_close(S, ref, RTOL[storage])
    assert ok, f"worst error / bound = {worst}"
    # the reference's own multi-mm / einsum decomposition gives the same matrix
    ref2 = ko.k_vs_all_scores_ref_form(model, Ev, Rv, hr, **kw)
    ok, worst = score_close(S, ref2, RTOL[storage])
    assert ok, worst


def _expected_counts(S_raw, targets, filters):
    out = np.array([ko.filtered_rank_counts(S_raw[j], int(targets[j]), filters[j]) for j in range(len(targets))])
    return out[:, 0], out[:, 1], out[:, 2]


@pytest.mark.parametrize("model,N,R,d,B,storage,kw", SCORE_CASES)
def test_rank_filtered_exact_against_own_scores(ops, FilterCSR, model, N, R, d, B, storage, kw):
    rng, hr, Eg, scg, Q, bias, Ev, Rv = _setup(ops, model, N, R, d, B, storage, kw, seed=1)
    targets = rng.integers(0, N, B).astype(np.int64)
    er = random_csr(rng, hr, targets, N, R)
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    hr_g = dev(torch.from_numpy(hr))
    rows = csr.rows_for(hr_g)
    out = ops.rank_filtered(Q, bias, Eg, scg, dev(torch.from_numpy(targets)), rows, csr.row_ptr, csr.col)
    S_raw = ops.scores(Q, None, Eg, scg).cpu().numpy()
    filters = [er[(int(h), int(r))] for h, r in hr]
    g, t, tl = _expected_counts(S_raw, targets, filters)
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)
    ts = out["target_score"].cpu().numpy()
    want_ts = S_raw[np.arange(B), targets] + bias.cpu().numpy()
    np.testing.assert_array_equal(ts, want_ts.astype(np.float32))
    # and inside the fp64 oracle's tolerance interval
    ref = ko.k_vs_all_scores(model, Ev, Rv, hr, **kw) - ko.build_query(model, Ev, Rv, hr, **kw)[1][:, None]
    ranks = 1 + g + tl
    for j in range(B):
        tol = RTOL[storage] * max(abs(ref[j, targets[j]]), np.sqrt((ref[j] ** 2).mean()))
        lo, hi = ko.rank_interval_with_tolerance(ref[j], int(targets[j]), filters[j], tol)
        assert lo <= ranks[j] <= hi


@pytest.mark.parametrize("storage,d", [("fp32", 40), ("bf16", 128), ("int8", 64)])
def test_rank_hub_rows_shared_filters_and_ties(ops, FilterCSR, storage, d):
    """Long filter rows (several slices and passes of the correction kernel), many queries sharing one
    (h, r) row, duplicated / zero entity rows (exact ties), unknown (h, r) pairs and no filter at all."""
    rng = np.random.default_rng(5)
    N, R, B = 9000, 3, 700
    E, Rel = random_tables(rng, N, R, d)
    E[100] = E[7000] = E[42]            # exact duplicates -> exact ties
    E[200:210] = 0.0                    # zero rows tie with each other
    hr = random_hr(rng, 40, R, B)       # few distinct pairs: big groups
    hr[:300] = hr[0]                    # one group of 300 queries
    targets = rng.integers(0, N, B).astype(np.int64)
    targets[:50] = 42
    targets[50:80] = 7000
    targets[80:100] = 205
    er = random_csr(rng, hr, targets, N, R, max_len=3, hub_rows=[(0, 5000), (400, 2500)])
    some = (int(hr[650, 0]), int(hr[650, 1]))
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Eg, scg = dev(Et), dev(sc)
    hr_g = dev(torch.from_numpy(hr))
    Q, bias = ops.build_query("DistMult", Eg, dev(Rt), hr_g, ent_scale=scg)
    csr = FilterCSR.from_er_vocab({k: v for k, v in er.items() if k != some}, R, device="cuda")
    rows = csr.rows_for(hr_g)
    assert int((rows < 0).sum()) > 0
    tg = dev(torch.from_numpy(targets))
    out = ops.rank_filtered(Q, bias, Eg, scg, tg, rows, csr.row_ptr, csr.col)
    S_raw = ops.scores(Q, None, Eg, scg).cpu().numpy()
    filters = [er[(int(h), int(r))] if (int(h), int(r)) != some else [] for h, r in hr]
    g, t, tl = _expected_counts(S_raw, targets, filters)
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)
    # no filter at all
    out2 = ops.rank_filtered(Q, bias, Eg, scg, tg)
    g2, t2, tl2 = _expected_counts(S_raw, targets, [None] * B)
    np.testing.assert_array_equal(out2["n_greater"].cpu().numpy(), g2)
    np.testing.assert_array_equal(out2["n_equal"].cpu().numpy(), t2)
    np.testing.assert_array_equal(out2["n_equal_lower"].cpu().numpy(), tl2)
    assert t2[:50].min() >= 2 and t2[80:100].min() >= 9        # duplicated / zero rows really tie


def test_rank_all_scores_equal(ops):
    """Zero embeddings: every score ties, the rank interval is [1, N]."""
    N, R, d, B = 500, 2, 32, 9
    E = torch.zeros((N, d), device="cuda")
    Rel = torch.zeros((R, d), device="cuda")
    hr = torch.zeros((B, 2), dtype=torch.int64, device="cuda")
    t = torch.arange(B, dtype=torch.int64, device="cuda") * 50
    Q, bias = ops.build_query("DistMult", E, Rel, hr)
    out = ops.rank_filtered(Q, bias, E, None, t)
    assert out["n_greater"].abs().max().item() == 0
    assert (out["n_equal"] == N - 1).all()
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), np.arange(B) * 50)


@pytest.mark.parametrize("storage,d", [("fp32", 48), ("bf16", 128), ("bf16", 64), ("int8", 128)])
def test_rank_one_filter_row_shared_by_different_query_vectors(ops, FilterCSR, storage, d):
    """The ABI takes Q and csr_row separately: queries may share a filter row without sharing a query vector
    (a range constraint per relation, a custom mask).  Each query must be corrected with ITS OWN scores of the
    filtered entities.  Rows: one long row shared by many distinct vectors, rows shared by a few, groups that mix
    repeated and distinct vectors, -1 (no filter)."""
    rng = np.random.default_rng(77)
    N, B = 6000, 900
    E = (rng.standard_normal((N, d)) * 0.1).astype(np.float32)
    Qh = (rng.standard_normal((B, d)) * 0.1).astype(np.float32)
    Qh[100:160] = Qh[100]                      # 60 queries with one vector ...
    Qh[160:170] = Qh[160]                      # ... and 10 with another, all on one row below
    Qh[170, 3] = 0.0
    Qh[171] = Qh[170]
    Qh[171, 3] = -0.0                          # equal values, different bits: its own round, same counts
    lens = [3000, 40, 7, 1, 0, 300, 2100]
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    col = np.concatenate([np.sort(rng.choice(N, size=n, replace=False)) for n in lens]).astype(np.int32)
    csr_row = rng.integers(-1, len(lens), B).astype(np.int64)
    csr_row[:60] = 0                           # 60 distinct vectors on the long row
    csr_row[100:172] = 6                       # the mixed group
    targets = rng.integers(0, N, B).astype(np.int64)
    targets[:20] = col[:20]                    # targets inside their own filter row stay unfiltered
    Et, sc, _, _, _ = stored_tables(E, E[:1], storage)
    Eg, scg, Qg = dev(Et), dev(sc), dev(torch.from_numpy(Qh))
    out = ops.rank_filtered(Qg, None, Eg, scg, dev(torch.from_numpy(targets)), dev(torch.from_numpy(csr_row)),
                            dev(torch.from_numpy(row_ptr)), dev(torch.from_numpy(col)))
    S_raw = ops.scores(Qg, None, Eg, scg).cpu().numpy()
    filters = [col[row_ptr[r]:row_ptr[r + 1]] if r >= 0 else None for r in csr_row]
    g, t, tl = _expected_counts(S_raw, targets, filters)
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)


@pytest.mark.parametrize("storage,d", [("fp32", 50), ("bf16", 128), ("bf16", 256), ("int8", 128)])
def test_rank_with_hoisted_thresholds_equals_the_plain_call(ops, FilterCSR, storage, d):
    """One threshold launch over all queries, then the rank in batches against slices of its result
    (the evaluator's grouping, reference evaluator.py:484-508 processes the same batches one by one): counters and
    target scores identical to ``rank_filtered`` over all queries at once.  With ``one_vector_per_row`` (rows and
    vectors from the same (h, r) pairs) and without it (vectors that share a row but differ)."""
    rng = np.random.default_rng(901 + d)
    N, R, B, bs = 7000, 4, 1100, 256
    E, Rel = random_tables(rng, N, R, d)
    E[11] = E[12]                                   # an exact tie
    hr = random_hr(rng, 60, R, B)
    targets = rng.integers(0, N, B).astype(np.int64)
    targets[:40] = 11
    er = random_csr(rng, hr, targets, N, R, max_len=5, hub_rows=[(0, 3000)])
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Eg, scg = dev(Et), dev(sc)
    hr_g = dev(torch.from_numpy(hr))
    tg = dev(torch.from_numpy(targets))
    Q, _ = ops.build_query("DistMult", Eg, dev(Rt), hr_g, ent_scale=scg)
    bias = dev(torch.from_numpy(rng.standard_normal(B).astype(np.float32)))
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    rows = csr.rows_for(hr_g)
    for same_vectors in (True, False):
        if not same_vectors:
            Q = Q.clone()
            Q[::3] += dev(torch.from_numpy((rng.standard_normal((len(range(0, B, 3)), d)) * 0.01).astype(np.float32)))
        want = ops.rank_filtered(Q, bias, Eg, scg, tg, rows, csr.row_ptr, csr.col)
        got = {k: torch.full((B,), -7, dtype=v.dtype, device="cuda") for k, v in want.items()}
        thr = ops.rank_thresholds(Q, bias, Eg, scg, tg, got)
        np.testing.assert_array_equal(got["target_score"].cpu().numpy(), want["target_score"].cpu().numpy())
        for i in range(0, B, bs):
            sl = slice(i, min(i + bs, B))
            Qi = Q[sl] if Q[sl].data_ptr() % 16 == 0 else Q[sl].clone()
            ops.rank_filtered(Qi, None, Eg, scg, tg[sl], rows[sl], csr.row_ptr, csr.col,
                              out={k: v[sl] for k, v in got.items()}, thr=thr[sl], one_vector_per_row=same_vectors)
        for k in want:
            np.testing.assert_array_equal(got[k].cpu().numpy(), want[k].cpu().numpy(), err_msg=f"{k} {same_vectors}")
    with pytest.raises(ValueError):
        ops.rank_filtered(Q, None, Eg, scg, tg, rows, csr.row_ptr, csr.col, thr=thr)      # thr= without out=


@pytest.mark.parametrize("storage,d,N", [("bf16", 64, 4097), ("fp32", 1, 1000), ("fp32", 32, 3001), ("bf16", 128, 5000),
                                         ("int8", 128, 2500), ("bf16", 256, 1300), ("bf16", 256, 40000),
                                         ("bf16", 200, 40000), ("int8", 192, 2500), ("bf16", 512, 40000),
                                         ("bf16", 328, 2500), ("int8", 448, 2500)])
def test_rank_partial_last_query_group_with_a_bias(ops, FilterCSR, storage, d, N):
    """B = 2500 leaves the last query group of every main loop partly filled (256-, 512- and 128-query groups), and
    the per-query bias is non-zero: ranks compare un-biased scores, target_score carries the bias."""
    rng = np.random.default_rng(1234 + d)
    R, B = 7, 2500
    E, Rel = random_tables(rng, N, R, d)
    hr = random_hr(rng, N, R, B)
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Eg, scg = dev(Et), dev(sc)
    hr_g = dev(torch.from_numpy(hr))
    Q, _ = ops.build_query("DistMult", Eg, dev(Rt), hr_g, ent_scale=scg)
    bias = dev(torch.from_numpy((rng.standard_normal(B) * 3.0).astype(np.float32)))
    targets = rng.integers(0, N, B).astype(np.int64)
    er = random_csr(rng, hr, targets, N, R, max_len=4)
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    out = ops.rank_filtered(Q, bias, Eg, scg, dev(torch.from_numpy(targets)), csr.rows_for(hr_g), csr.row_ptr, csr.col)
    S_raw = ops.scores(Q, None, Eg, scg).cpu().numpy()
    filters = [er[(int(h), int(r))] for h, r in hr]
    g, t, tl = _expected_counts(S_raw, targets, filters)
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)
    want_ts = (S_raw[np.arange(B), targets] + bias.cpu().numpy()).astype(np.float32)
    np.testing.assert_array_equal(out["target_score"].cpu().numpy(), want_ts)
    # the biased matrix: same bits as raw + bias, rounded once
    S_b = ops.scores(Q, bias, Eg, scg).cpu().numpy()
    np.testing.assert_array_equal(S_b, (S_raw + bias.cpu().numpy()[:, None]).astype(np.float32))


def test_rank_of_more_queries_than_one_launch_of_the_four_tile_kernel_takes(ops):
    """bf16, d = 128, B = 40,000: the four-tile rank kernel is launched per 16,384 queries (two full launches and a
    ragged third); counters, without a filter, against torch reductions of the library's own score matrix, on the GPU."""
    g = torch.Generator(device="cuda").manual_seed(77)
    N, d, B = 1500, 128, 40000
    E = (torch.randn((N, d), device="cuda", generator=g) * 0.3).to(torch.bfloat16).contiguous()
    E[7] = E[3]                                    # ties
    Q = torch.randn((B, d), device="cuda", generator=g) * 0.3
    tgt = torch.randint(0, N, (B,), device="cuda", generator=g)
    tgt[::5] = 3
    out = ops.rank_filtered(Q, None, E, None, tgt)
    S = ops.scores(Q, None, E, None)
    thr = S[torch.arange(B, device="cuda"), tgt]
    assert torch.equal(out["target_score"], thr)
    assert torch.equal(out["n_greater"], (S > thr[:, None]).sum(1).int())
    eq = S == thr[:, None]
    assert torch.equal(out["n_equal"], eq.sum(1).int() - 1)
    lower = torch.arange(N, device="cuda")[None, :] < tgt[:, None]
    assert torch.equal(out["n_equal_lower"], (eq & lower).sum(1).int())
    assert int(out["n_equal"].max()) >= 1


@pytest.mark.parametrize("sq,se", [(1e-6, 1e-6), (1e6, 1e6), (1e-12, 1e-3), (1e-15, 1e-15), (3e17, 3e17), (1e-30, 1.0)])
def test_fp32_scores_hold_their_accuracy_across_magnitudes(ops, sq, se):
    """fp32 tables run as three bf16 parts per operand.  Inside the documented range (every product q*e of a score
    at least 2^-100 in magnitude and every value's bf16 rounding finite) the scores stay within 1e-5 of fp64."""
    rng = np.random.default_rng(5)
    N, d, B = 700, 200, 130
    E = (rng.standard_normal((N, d)) * se).astype(np.float32)
    Qh = (rng.standard_normal((B, d)) * sq).astype(np.float32)
    S = ops.scores(dev(torch.from_numpy(Qh)), None, dev(torch.from_numpy(E)), None).cpu().numpy()
    ref = Qh.astype(np.float64) @ E.astype(np.float64).T
    ok, worst = score_close(S, ref, 1e-5)
    assert ok, worst


def test_fp32_scores_below_the_documented_range_degrade_gracefully(ops):
    """Products near the bottom of fp32's range (|q*e| ~ 1e-36): the low-order parts underflow, the leading bf16
    products remain, so the result is still a bf16-grade score (2e-2), never garbage; products that underflow fp32
    altogether give exact zeros, as fp32 arithmetic itself would."""
    rng = np.random.default_rng(6)
    N, d, B = 300, 64, 40
    E = (rng.standard_normal((N, d)) * 1e-18).astype(np.float32)
    Qh = (rng.standard_normal((B, d)) * 1e-18).astype(np.float32)
    S = ops.scores(dev(torch.from_numpy(Qh)), None, dev(torch.from_numpy(E)), None).cpu().numpy()
    ref = Qh.astype(np.float64) @ E.astype(np.float64).T
    ok, worst = score_close(S, ref, 2e-2)
    assert ok, worst
    tiny = (rng.standard_normal((N, d)) * 1e-30).astype(np.float32)
    S0 = ops.scores(dev(torch.from_numpy(tiny[:B].copy())), None, dev(torch.from_numpy(tiny)), None).cpu().numpy()
    assert np.all(S0 == 0.0)


TOPK_CASES = [
    ("DistMult", 135, 46, 32, 64, "fp32", 10),
    ("ComplEx", 20011, 11, 200, 130, "fp32", 100),
    ("QMult", 20011, 5, 128, 600, "bf16", 10),
    ("DistMult", 30000, 9, 128, 70, "int8", 100),
    ("DistMult", 9000, 9, 192, 70, "int8", 50),      # int8 wider than 128
    ("DistMult", 9000, 9, 512, 70, "bf16", 50),      # bf16 wider than 256: four segments of 128 columns
    ("DistMult", 9000, 9, 512, 70, "int8", 50),      # int8 likewise
    ("DistMult", 5000, 9, 320, 300, "bf16", 10),     # ... three, the last one partly zero
    ("DistMult", 5000, 9, 64, 33, "bf16", 1),
    ("DistMult", 6000, 9, 64, 20, "fp32", 1024),
    ("DistMult", 700, 9, 64, 20, "fp32", 600),       # k above half of the one-wave select's capacity
    ("DistMult", 1000, 9, 32, 10, "fp32", 1000),     # k == N
    ("DistMult", 3000, 5, 64, 40, "bf16", 300),
    ("ComplEx", 9000, 5, 64, 24, "fp32", 511),
]


@pytest.mark.parametrize("N,B,k,pattern", [(150001, 1100, 10, "random"), (70001, 2500, 100, "random"),
                                           (140000, 1024, 10, "ties"), (131072, 900, 1, "best_last"),
                                           (98304 + 17, 1030, 300, "random")])
def test_topk_bf16_d128_long_rounds_equal_the_materialised_scores(ops, N, B, k, pattern):
    """bf16 tables with d = 128, batches of a thousand queries and more, tables long enough for rounds of tens of
    thousands of rows (the persistent scan with several chunks per workgroup).  Values and indices against the
    library's own scores, ties towards the lower id; tables with thousands of exact ties, with the best rows at the
    very end (every round collects), a partial last stage and a partial last query group."""
    rng = np.random.default_rng(N + B + k)
    d = 128
    E = (rng.standard_normal((N, d)) * 0.1).astype(np.float32)
    if pattern == "ties":
        pool = (rng.standard_normal((7, d)) * 0.1).astype(np.float32)
        E[rng.integers(0, N, N // 3)] = pool[rng.integers(0, 7, N // 3)]
        E[N - 5000:] = pool[0]
    if pattern == "best_last":
        E *= np.linspace(0.2, 3.0, N, dtype=np.float32)[:, None]
    Q = (rng.standard_normal((B, d)) * 0.1).astype(np.float32)
    Q[3] = 0.0
    Eg = dev(torch.from_numpy(E)).to(torch.bfloat16).contiguous()
    Qg = dev(torch.from_numpy(Q))
    bias = dev(torch.from_numpy(rng.standard_normal(B).astype(np.float32)))
    vals, idx = ops.topk(Qg, bias, Eg, None, k)
    # (the order is that of the scores before the bias, which is the same for every entity of a query: two raw scores
    # that differ can round to one value once it is added)
    S_raw = ops.scores(Qg, None, Eg, None).cpu().numpy()
    wv, wi = ko.topk(S_raw, k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), (wv + bias.cpu().numpy()[:, None]).astype(np.float32))


@pytest.mark.parametrize("model,N,R,d,B,storage,k", TOPK_CASES)
def test_topk_exact_against_own_scores(ops, model, N, R, d, B, storage, k):
    rng, hr, Eg, scg, Q, bias, Ev, Rv = _setup(ops, model, N, R, d, B, storage, {}, seed=2)
    vals, idx = ops.topk(Q, bias, Eg, scg, k)
    S = ops.scores(Q, bias, Eg, scg).cpu().numpy()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)
    # sigmoid variant equals sigmoid of the logits at the same entities
    sv, si = ops.topk(Q, bias, Eg, scg, k, sigmoid=True)
    np.testing.assert_array_equal(si.cpu().numpy(), wi)
    np.testing.assert_allclose(sv.cpu().numpy(), ko.sigmoid(wv), rtol=1e-6, atol=1e-7)
    # against the fp64 oracle: same index set wherever the k-th / (k+1)-th gap exceeds tolerance
    ref = ko.k_vs_all_scores(model, Ev, Rv, hr)
    for b in range(B):
        order = np.argsort(-ref[b], kind="stable")
        tol = RTOL[storage] * np.sqrt((ref[b] ** 2).mean())
        if k < N and ref[b, order[k - 1]] - ref[b, order[k]] > 2 * tol:
            assert set(order[:k]) == set(wi[b])


def test_topk_adversarial_order_overflows_and_recovers(ops):
    """Scores that increase with the entity id defeat the running threshold: every new row beats it,
    the candidate buffers overflow and the rescan path has to repair the result."""
    N, d, B, k = 60000, 16, 40, 10
    rng = np.random.default_rng(3)
    v = rng.standard_normal(d).astype(np.float32)
    E = (np.arange(N, dtype=np.float32)[:, None] / N) * v[None, :]
    Q = (np.abs(rng.standard_normal((B, 1))).astype(np.float32) + 0.5) * v[None, :]
    Eg, Qg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Q))
    vals, idx = ops.topk(Qg, None, Eg, None, k)
    S = ops.scores(Qg, None, Eg, None).cpu().numpy()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)


@pytest.mark.parametrize("storage", ["fp32", "int8"])
def test_topk_best_rows_first_defeats_the_guessed_threshold(ops, storage):
    """Scores that decrease with the entity id: the best k are all in the first round, so the threshold a later scan
    guesses from the order statistics of a shuffled table (a rank above the k-th) is too high every time.  The
    selection notices that fewer than k entries beat the guess, flags the query, and the final rescan with the k-th
    best repairs it."""
    N, d, B, k = 70000, 128, 70, 100
    rng = np.random.default_rng(5)
    v = rng.standard_normal(d).astype(np.float32)
    E = ((N - np.arange(N, dtype=np.float32))[:, None] / N) * v[None, :]
    E += (rng.standard_normal((N, d)) * 1e-4).astype(np.float32)
    Q = (np.abs(rng.standard_normal((B, 1))).astype(np.float32) + 0.5) * v[None, :]
    Et, sc, _, _, _ = stored_tables(E, E[:1], storage)
    Eg, scg, Qg = dev(Et), dev(sc), dev(torch.from_numpy(Q))
    vals, idx = ops.topk(Qg, None, Eg, scg, k)
    S = ops.scores(Qg, None, Eg, scg).cpu().numpy()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)


@pytest.mark.parametrize("N,B,k", [(70001, 1100, 100), (200003, 33, 1), (150000, 40, 1024), (4100, 20, 10)])
def test_topk_int8_filter_scan_edge_cases(ops, N, B, k):
    """The int8 scan admits candidates by an integer bound and scores them exactly afterwards; whatever the bound
    lets through or not, the result must be the top k of the library's own scores.  Rows: scales spread over four
    orders of magnitude, zero and negative scales, scales so small that their reciprocal overflows, all-zero rows,
    rows of +-127; queries: zero, one-hot, a huge dynamic range, one whose scores are all negative, one of components
    around 1e34 (beyond the range in which the bound's arithmetic stays finite: every row becomes a candidate), one
    of components around 1e-36; N not a multiple of the 64-row stage, a partial last query group."""
    rng = np.random.default_rng(N + k)
    d = 128
    q8 = rng.integers(-127, 128, (N, d)).astype(np.int8)
    q8[rng.integers(0, N, 50)] = 0
    q8[rng.integers(0, N, 50)] = 127
    q8[rng.integers(0, N, 50)] = -127
    sc = np.exp(rng.uniform(np.log(1e-5), np.log(1e-1), N)).astype(np.float32)
    sc[rng.integers(0, N, 200)] = 0.0
    neg = rng.integers(0, N, 200)
    sc[neg] = -sc[neg]
    sc[rng.integers(0, N, 100)] = 1e-40                # 1 / scale is infinite in fp32
    sc[N // 2 - 100:N // 2 + 100] = 2e-39              # whole tiles of them
    Q = (rng.standard_normal((B, d)) * 0.1).astype(np.float32)
    Q[0] = 0.0
    Q[1] = 0.0
    Q[1, 5] = 3.0
    Q[2] *= np.exp(rng.uniform(-12, 2, d)).astype(np.float32)
    base = np.abs(rng.standard_normal(d)).astype(np.float32)
    Q[3] = -base                                       # against rows made non-negative below: every score <= 0
    Q[4] *= 2e35
    Q[5] *= 1e-35
    Eg, scg, Qg = dev(torch.from_numpy(q8)), dev(torch.from_numpy(sc)), dev(torch.from_numpy(Q))
    vals, idx = ops.topk(Qg, None, Eg, scg, k)
    S = ops.scores(Qg, None, Eg, scg).cpu().numpy()
    wv, wi = ko.topk(S, k)
    # (the zero query scores +0 or -0 everywhere: equal to numpy, ordered by sign in the library's keys)
    np.testing.assert_array_equal(idx.cpu().numpy()[1:], wi[1:])
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)
    # the table's derived form made once and handed in: the same bits, on two calls that share it
    prep = ops.topk_prepare(Eg, scg)
    assert prep is not None and prep.numel() >= N * d
    for _ in range(2):
        v2, i2 = ops.topk(Qg, None, Eg, scg, k, prepared=prep)
        assert torch.equal(v2, vals) and torch.equal(i2, idx)
    # a table of non-negative rows and positive scales under the all-negative query
    Ep = np.abs(q8.astype(np.int16)).clip(0, 127).astype(np.int8)
    scp = np.abs(sc) + 1e-6
    Eg, scg = dev(torch.from_numpy(Ep)), dev(torch.from_numpy(scp))
    vals, idx = ops.topk(Qg[3:4], None, Eg, scg, k)
    S = ops.scores(Qg[3:4], None, Eg, scg).cpu().numpy()
    assert (S <= 0).all()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)


def test_topk_prepared_form_exists_for_int8_d128_only(ops):
    from dicee_amd import _lib
    lib = _lib.load()
    assert lib.kge_topk_prepared_bytes(2, 128, 1000) >= 1000 * 128 + 16 * 32
    assert lib.kge_topk_prepared_bytes(2, 64, 1000) == 0 and lib.kge_topk_prepared_bytes(1, 128, 1000) == 0
    assert lib.kge_topk_prepared_bytes(0, 128, 1000) == 0
    E = torch.zeros((1000, 64), dtype=torch.int8, device="cuda")
    sc = torch.ones(1000, device="cuda")
    assert ops.topk_prepare(E, sc) is None
    assert ops.topk_prepare(torch.zeros((1000, 128), dtype=torch.bfloat16, device="cuda"), None) is None
    p256 = ctypes.c_void_p(256)
    assert lib.kge_topk_prepare(p256, 1, p256, 128, 1000, p256, 1 << 30, None) == 2        # bf16: no prepared form
    assert lib.kge_topk_prepare(p256, 2, p256, 128, 1000, p256, 100, None) == 3            # buffer too small
    assert b"need" in lib.kge_last_error()
    assert lib.kge_topk_prepared(p256, None, p256, 2, p256, 4, 128, 1000, 5, p256, p256, 0, p256, 100, p256, 1 << 30,
                                 None) == 3                                                  # prepared too small
    assert lib.kge_topk_prepared(p256, None, p256, 2, p256, 4, 64, 1000, 5, p256, p256, 0, p256, 1 << 30, p256, 1 << 30,
                                 None) == 2                                                  # d = 64: call kge_topk
    # a small table (one round, no filter scan) accepts a prepared buffer and ignores it
    E8 = torch.randint(-127, 128, (500, 128), dtype=torch.int8, device="cuda")
    s8 = torch.full((500,), 0.02, device="cuda")
    Q = torch.randn((7, 128), device="cuda")
    prep = ops.topk_prepare(E8, s8)
    v1, i1 = ops.topk(Q, None, E8, s8, 9)
    v2, i2 = ops.topk(Q, None, E8, s8, 9, prepared=prep)
    assert torch.equal(v1, v2) and torch.equal(i1, i2)


def test_topk_int8_query_with_a_nan_yields_nothing(ops):
    N, d, B, k = 9000, 128, 3, 5
    rng = np.random.default_rng(8)
    q8 = rng.integers(-127, 128, (N, d)).astype(np.int8)
    sc = np.full(N, 0.01, dtype=np.float32)
    Q = rng.standard_normal((B, d)).astype(np.float32)
    Q[1, 17] = np.nan
    vals, idx = ops.topk(dev(torch.from_numpy(Q)), None, dev(torch.from_numpy(q8)), dev(torch.from_numpy(sc)), k)
    assert torch.isnan(vals[1]).all() and (idx[1] == -1).all()
    S = ops.scores(dev(torch.from_numpy(Q[[0, 2]])), None, dev(torch.from_numpy(q8)), dev(torch.from_numpy(sc))).cpu().numpy()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(idx[[0, 2]].cpu().numpy(), wi)


def test_topk_ties_prefer_lower_ids_and_k_equals_n(ops):
    N, d, B = 300, 16, 5
    E = torch.zeros((N, d), device="cuda")
    Q = torch.ones((B, d), device="cuda")
    vals, idx = ops.topk(Q, None, E, None, 7)
    np.testing.assert_array_equal(idx.cpu().numpy(), np.tile(np.arange(7), (B, 1)))
    vals, idx = ops.topk(Q, None, E, None, N)
    np.testing.assert_array_equal(idx.cpu().numpy(), np.tile(np.arange(N), (B, 1)))


@pytest.mark.parametrize("storage", ["fp32", "bf16", "int8"])
@pytest.mark.parametrize("k", [1, 3, 100])
@pytest.mark.parametrize("best_value", [90, 0])
def test_topk_many_ties_at_the_top_survive_an_overflowing_round(ops, storage, k, best_value):
    """Thousands of entities share the best score, and all of them fall into one round, whose candidate buffer
    (4096 slots) overflows and keeps a random sample.  The repair scan must bring back the ties with the LOWEST ids,
    which no score threshold can tell from the others: it admits by key (score, then entity id).  With best_value 0
    the shared score is +0.0, whose neighbour in the ordered encoding (-0.0) compares equal to it."""
    rng = np.random.default_rng(77 + k)
    N, d, B = 60000, 128, 6
    q = np.zeros((B, d), dtype=np.float32)
    q[:, :8] = 1.0
    lo = rng.integers(-40, 0, (N, d)).astype(np.int8)              # every ordinary row scores below zero
    tied = np.sort(rng.choice(np.arange(1100, 16000), 9000, replace=False))
    best = np.zeros(d, dtype=np.int8)
    best[:8] = best_value
    lo[tied] = best                                                  # 9000 identical rows: one exact score
    if storage == "int8":
        E = dev(torch.from_numpy(lo))
        sc = dev(torch.full((N,), 0.01))
    else:
        E = dev(torch.from_numpy(lo.astype(np.float32) * 0.01))
        sc = None
        if storage == "bf16":
            E = E.to(torch.bfloat16)
    Qg = dev(torch.from_numpy(q))
    vals, idx = ops.topk(Qg, None, E, sc, k)
    S = ops.scores(Qg, None, E, sc).cpu().numpy()
    assert (S[:, tied] == S[0, tied[0]]).all() and S[0, tied[0]] == S.max()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)
    np.testing.assert_array_equal(idx.cpu().numpy()[0], tied[:k])


@pytest.mark.parametrize("model,N,R,d,B,storage,kw", [
    ("Keci", 4099, 18, 256, 300, "fp32", {"p": 0, "q": 1, "coeff_q": [1.0]}),
    ("Keci", 1000, 6, 35, 70, "fp32", {"p": 3, "q": 3, "coeff_p": [0.7, 1.1, -0.3], "coeff_q": [1.3, -0.4, 0.9]}),
    ("QMult", 3000, 5, 128, 530, "bf16", {}),
    ("DistMult", 2000, 5, 64, 100, "int8", {}),
    ("DistMult", 1100, 5, 160, 100, "int8", {}),
    ("ComplEx", 3000, 5, 200, 530, "bf16", {}),
    ("DistMult", 3000, 5, 448, 300, "bf16", {}),
])
@pytest.mark.parametrize("eps", [0.0, 0.1])
def test_bce_multihot_vs_oracle(ops, FilterCSR, model, N, R, d, B, storage, kw, eps):
    rng, hr, Eg, scg, Q, bias, Ev, Rv = _setup(ops, model, N, R, d, B, storage, kw, seed=4, std=0.5)
    er = random_csr(rng, hr, rng.integers(0, N, B), N, R, max_len=5, hub_rows=[(0, 400)])
    er[(int(hr[1, 0]), int(hr[1, 1]))] = er.get((int(hr[1, 0]), int(hr[1, 1])), [])
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    rows = csr.rows_for(dev(torch.from_numpy(hr)))
    loss = ops.bce_multihot(Q, bias, Eg, scg, rows, csr.row_ptr, csr.col, eps).item()
    ref = ko.k_vs_all_scores(model, Ev, Rv, hr, **kw)
    want = ko.bce_multihot(ref, [er[(int(h), int(r))] for h, r in hr], eps)
    tol = 1e-5 if storage == "fp32" else 2e-2
    assert loss == pytest.approx(want, rel=tol)


@pytest.mark.parametrize("model,N,R,d,B,kw", [
    ("Keci", 4099, 18, 256, 300, {"p": 0, "q": 1, "coeff_q": [1.0]}),
    ("Keci", 1000, 6, 35, 70, {"p": 3, "q": 3, "coeff_p": [0.7, 1.1, -0.3], "coeff_q": [1.3, -0.4, 0.9]}),
    ("DistMult", 777, 5, 64, 1, {}),
    ("ComplEx", 130, 5, 200, 513, {}),
    ("DistMult", 40, 3, 7, 33, {}),
    # widths that are multiples of 4 take the gradient contractions with K-major operands: a second entity tile of
    # four rows, a single quad, several K splits with a ragged last one on both products
    ("DistMult", 1000, 5, 260, 130, {}),
    ("DistMult", 37, 3, 4, 2, {}),
    ("ComplEx", 5003, 5, 512, 2100, {}),
])
@pytest.mark.parametrize("eps", [0.0, 0.1])
def test_bce_backward_vs_oracle(ops, FilterCSR, model, N, R, d, B, kw, eps):
    """dQ, dbias and dE of the fused BCE step against the fp64 closed form (sigmoid(S) - y') / (B N) pushed
    through the two products.  Tolerance 1e-5 of each gradient's RMS (sums of up to N resp. B fp32 terms)."""
    rng, hr, Eg, scg, Q, bias, Ev, Rv = _setup(ops, model, N, R, d, B, "fp32", kw, seed=6, std=0.5)
    er = random_csr(rng, hr, rng.integers(0, N, B), N, R, max_len=5, hub_rows=[(0, min(400, N // 2))])
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    rows = csr.rows_for(dev(torch.from_numpy(hr)))
    loss, dQ, dbias, dE = ops.bce_multihot_backward(Q, bias, Eg, rows, csr.row_ptr, csr.col, eps, grad_out=1.5)
    fwd = ops.bce_multihot(Q, bias, Eg, None, rows, csr.row_ptr, csr.col, eps)
    assert loss.item() == pytest.approx(fwd.item(), rel=1e-6)
    Qr, br = ko.build_query(model, Ev, Rv, hr, **kw)
    positives = [er.get((int(h), int(r)), []) for h, r in hr]
    wQ, wb, wE = ko.bce_multihot_backward(Qr, br, Ev, positives, eps, grad_out=1.5)
    for got, want, name in ((dQ, wQ, "dQ"), (dE, wE, "dE")):
        got = got.cpu().numpy()
        assert got.shape == want.shape and np.isfinite(got).all(), name
        rms = np.sqrt((want ** 2).mean())
        assert np.abs(got - want).max() <= 1e-5 * rms + 1e-12, (name, np.abs(got - want).max() / rms)
    # a row sum of the score gradient cancels (sigmoid part against the known tails): bound by the sum of magnitudes
    S = Qr @ Ev.T + br[:, None]
    g_abs = 1.5 * (ko.sigmoid(S) + ko.dense_multihot(positives, N, eps, dtype=np.float64)) / (B * N)
    got = dbias.cpu().numpy()
    assert got.shape == wb.shape
    assert np.all(np.abs(got - wb) <= 2e-6 * g_abs.sum(axis=1)), np.max(np.abs(got - wb) / g_abs.sum(axis=1))


def test_bce_backward_argument_checks(ops):
    from dicee_amd._lib import KgeError
    E = torch.zeros((64, 128), device="cuda", dtype=torch.bfloat16)
    Q = torch.zeros((4, 128), device="cuda")
    with pytest.raises(TypeError):
        ops.bce_multihot_backward(Q, None, E, None, None, None)
    lib = __import__("dicee_amd._lib", fromlist=["load"]).load()
    assert lib.kge_bce_backward_workspace_bytes(0, 8, 8) == 0
    rc = lib.kge_bce_multihot_backward(Q.data_ptr(), None, E.data_ptr(), 1, 4, 128, 64, None, None, None, 0, 0.0, 1.0,
                                       None, Q.data_ptr(), None, Q.data_ptr(), Q.data_ptr(), 1 << 20, None)
    assert rc == 2                                               # KGE_ERR_UNSUPPORTED: bf16 table


def test_argument_validation(ops):
    from dicee_amd._lib import KgeError
    E = torch.zeros((100, 24), device="cuda")
    Q = torch.zeros((4, 24), device="cuda")
    with pytest.raises(KgeError):
        ops.topk(Q, None, E, None, 101)                      # k > N
    with pytest.raises(KgeError):
        ops.topk(Q, None, E, None, 0)
    with pytest.raises(KgeError):
        ops.build_query("QMult", torch.zeros((10, 6), device="cuda"), torch.zeros((2, 6), device="cuda"),
                        torch.zeros((1, 2), dtype=torch.int64, device="cuda"))   # d % 4 != 0
    with pytest.raises(KgeError):
        ops.build_query("Keci", torch.zeros((10, 7), device="cuda"), torch.zeros((2, 7), device="cuda"),
                        torch.zeros((1, 2), dtype=torch.int64, device="cuda"), p=1, q=1,
                        coeff_p=torch.ones(1, device="cuda"), coeff_q=torch.ones(1, device="cuda"))
    with pytest.raises(KgeError):
        ops.scores(torch.zeros((4, 136), device="cuda"), None, torch.zeros((10, 136), device="cuda", dtype=torch.int8),
                   torch.ones(10, device="cuda"))                               # int8 with d % 16 != 0
    with pytest.raises(RuntimeError):
        ops.scores(torch.zeros((4, 24)), None, torch.zeros((10, 24)))            # CPU tensors
    # empty batch is a no-op
    out = ops.scores(torch.zeros((0, 24), device="cuda"), None, E)
    assert out.shape == (0, 100)


def test_rank_large_batch_spans_several_filter_plans(ops, FilterCSR):
    """B > 8192: the filter correction is planned per sub-batch of 8192 queries (the largest plan,
    which also needs the opt-in LDS size); one shared hub row, thousands of distinct rows."""
    rng = np.random.default_rng(11)
    N, R, d, B = 3000, 50, 64, 8192 + 700
    E, Rel = random_tables(rng, N, R, d)
    hr = random_hr(rng, N, R, B)
    hr[::7] = hr[0]
    targets = rng.integers(0, N, B).astype(np.int64)
    er = random_csr(rng, hr, targets, N, R, max_len=4, hub_rows=[(0, 2500)])
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, "bf16")
    Eg = dev(Et)
    hr_g = dev(torch.from_numpy(hr))
    Q, bias = ops.build_query("ComplEx", Eg, dev(Rt), hr_g)
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    out = ops.rank_filtered(Q, bias, Eg, None, dev(torch.from_numpy(targets)), csr.rows_for(hr_g), csr.row_ptr,
                            csr.col)
    S_raw = ops.scores(Q, None, Eg, None).cpu().numpy()
    g, t, tl = _expected_counts(S_raw, targets, [er[(int(h), int(r))] for h, r in hr])
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)


def test_plan_written_by_the_gpu_satisfies_the_host_model_invariants(ops, FilterCSR):
    """The plan of the filter correction as plan_fix_kernel leaves it in the workspace (layout and packed fields of
    csrc/kge_host.h, whose sequential model the CPU suite runs under sanitizers): groups partition the queries that
    have a non-empty filter row, member positions are contiguous, the work list covers every slice exactly once."""
    import ctypes
    from dicee_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(21)
    N, R, d, B = 3000, 5, 32, 3000
    E, Rel = random_tables(rng, N, R, d)
    hr = random_hr(rng, 300, R, B)
    hr[:500] = hr[0]
    targets = rng.integers(0, N, B).astype(np.int64)
    er = random_csr(rng, hr, targets, N, R, max_len=3, hub_rows=[(0, 2900), (700, 1500)])
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    Eg, hr_g = dev(torch.from_numpy(E)), dev(torch.from_numpy(hr))
    Q, bias = ops.build_query("DistMult", Eg, dev(torch.from_numpy(Rel)), hr_g)
    rows = csr.rows_for(hr_g)
    out = [torch.empty((B,), dtype=torch.int32, device="cuda") for _ in range(3)] + [torch.empty((B,), device="cuda")]
    ws_bytes = lib.kge_rank_workspace_bytes(B)
    ws = torch.zeros((ws_bytes,), dtype=torch.uint8, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.kge_rank_filtered(p(Q), p(bias), p(Eg), _lib.DTYPE_F32, None, B, d, N, p(dev(torch.from_numpy(targets))),
                               p(rows), p(csr.row_ptr), p(csr.col), csr.row_ptr.numel() - 1, p(out[0]), p(out[1]),
                               p(out[2]), p(out[3]), p(ws), ws_bytes, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.kge_last_error()
    torch.cuda.synchronize()
    up = lambda x: (x + 255) // 256 * 256
    SORT_MAX = 8192
    # thresholds, leaders, mixed-group flags (one int32 per query each), then one plan per 8192 queries
    o_lead = up(4 * B)
    o_mixed = o_lead + up(4 * B)
    o_skey = o_mixed + up(4 * B)
    o_gend = o_skey + up(8 * SORT_MAX)
    o_work = o_gend + up(4 * SORT_MAX)
    o_meta = o_work + up(8 * SORT_MAX)
    assert o_meta + 256 == ws_bytes
    raw = ws.cpu().numpy()
    skey = raw[o_skey:o_skey + 8 * SORT_MAX].view(np.uint64)
    gend = raw[o_gend:o_gend + 4 * SORT_MAX].view(np.int32)
    work = raw[o_work:o_work + 8 * SORT_MAX].view(np.int32).reshape(-1, 2)
    n_work, slice_len, n_groups = (int(v) for v in raw[o_meta:o_meta + 12].view(np.int32))
    lead = raw[o_lead:o_lead + 4 * B].view(np.int32)
    assert not raw[o_mixed:o_mixed + 4 * B].view(np.int32).any()
    rp = csr.row_ptr.cpu().numpy()
    rows_h = rows.cpu().numpy()
    want = {}
    for i, r in enumerate(rows_h):
        if r >= 0 and rp[r + 1] > rp[r]:
            want.setdefault(int(r), set()).add(i)
    assert n_groups == len(want) and slice_len >= 128 and slice_len % 32 == 0
    seen_work, seen_rows = 0, set()
    for g in range(n_groups):
        first, w0 = int(work[g, 0]), int(work[g, 1])
        assert w0 == seen_work
        end = int(gend[first])
        row = int(skey[first] >> np.uint64(24))
        assert row in want and row not in seen_rows
        seen_rows.add(row)
        members = {int(skey[i] & np.uint64(0xffffff)) for i in range(first, end)}
        assert all(int(skey[i] >> np.uint64(24)) == row for i in range(first, end))
        assert members == want[row]
        # every member knows the group's leader (the query at the group's first sorted position); no group mixes vectors
        assert all(int(lead[i]) == int(skey[first] & np.uint64(0xffffff)) for i in members)
        seen_work += -(-(int(rp[row + 1] - rp[row])) // slice_len)
    assert seen_work == n_work
    no_row = [i for i, r in enumerate(rows_h) if not (r >= 0 and rp[r + 1] > rp[r])]
    assert all(int(lead[i]) == -1 for i in no_row)


def test_csr_lookup_matches_host_search(ops, FilterCSR):
    rng = np.random.default_rng(12)
    N, R = 500, 7
    triples = np.stack([rng.integers(0, N, 3000), rng.integers(0, R, 3000), rng.integers(0, N, 3000)], axis=1)
    csr = FilterCSR.from_triples(triples, R, device="cuda")
    hr = np.stack([rng.integers(0, N + 20, 4000), rng.integers(0, R, 4000)], axis=1).astype(np.int64)
    got = csr.rows_for(dev(torch.from_numpy(hr))).cpu().numpy()
    np.testing.assert_array_equal(got, csr.rows_for_numpy(hr))
    assert (got < 0).any() and (got >= 0).any()
    empty = FilterCSR.from_triples(np.empty((0, 3), dtype=np.int64), R, device="cuda")
    assert (empty.rows_for(dev(torch.from_numpy(hr[:5]))).cpu().numpy() == -1).all()


# ---------------------------------------------------------------------------------------------
# vocabulary -> CSR on the GPU
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kind", ["er", "re", "ee"])
@pytest.mark.parametrize("n,N,R", [(1, 5, 3), (700, 40, 7), (60000, 3000, 11), (300000, 200000, 1300)])
def test_csr_build_matches_the_vocabulary_oracle(kind, n, N, R):
    from dicee_amd.csr import FilterCSR
    rng = np.random.default_rng(n + len(kind))
    t = np.stack([rng.integers(0, N, n), rng.integers(0, R, n), rng.integers(0, N, n)], axis=1)
    t[n // 2:] = t[:n - n // 2]                                          # half of the triples are duplicates
    hub = rng.random(n) < 0.2
    t[hub, 0], t[hub, 1] = 1 % N, 2 % R                                  # one long (h, r) row
    csr = FilterCSR.from_triples_gpu(torch.from_numpy(t).cuda(), N, R, kind=kind)
    rb = {"er": R, "re": N, "ee": N}[kind]
    keys, row_ptr, col = ko.vocab_csr(t, kind, rb)
    assert csr.keys.dtype == torch.int64 and csr.row_ptr.dtype == torch.int64 and csr.col.dtype == torch.int32
    np.testing.assert_array_equal(csr.keys.cpu().numpy(), keys)
    np.testing.assert_array_equal(csr.row_ptr.cpu().numpy(), row_ptr)
    np.testing.assert_array_equal(csr.col.cpu().numpy(), col)
    assert csr.num_rows == len(keys) and csr.nnz == len(col)
    a, b, _ = {"er": (0, 1, 2), "re": (1, 2, 0), "ee": (0, 2, 1)}[kind]
    rows = csr.rows_for(torch.from_numpy(np.ascontiguousarray(t[:50][:, [a, b]])).cuda()).cpu().numpy()
    np.testing.assert_array_equal(keys[rows], t[:50, a] * rb + t[:50, b])


def test_csr_build_edge_cases():
    from dicee_amd import ops
    from dicee_amd.csr import FilterCSR
    empty = FilterCSR.from_triples_gpu(torch.empty((0, 3), dtype=torch.int64, device="cuda"), 10, 3)
    assert empty.num_rows == 0 and empty.nnz == 0 and empty.row_ptr.tolist() == [0]
    t = torch.tensor([[1, 0, 2], [9, 0, 2], [1, 3, 2], [1, 0, -1], [1, 0, 2], [0, 2, 9]], device="cuda")
    keys, row_ptr, col, dropped = ops.csr_build(t, (0, 1, 2), (9, 3, 10))      # h = 9, r = 3 and t = -1 are out of range
    assert dropped == 3 and keys.tolist() == [2, 3] and row_ptr.tolist() == [0, 1, 2] and col.tolist() == [9, 2]
    with pytest.raises(ValueError):
        FilterCSR.from_triples_gpu(t, 9, 3)
    only_bad = torch.tensor([[50, 0, 0]], device="cuda")
    keys, row_ptr, col, dropped = ops.csr_build(only_bad, (0, 1, 2), (9, 3, 10))
    assert dropped == 1 and keys.numel() == 0 and row_ptr.tolist() == [0] and col.numel() == 0
    with pytest.raises(TypeError):
        ops.csr_build(t.int(), (0, 1, 2), (9, 3, 10))


def test_csr_built_on_the_gpu_filters_like_the_host_built_one():
    from dicee_amd import ops
    from dicee_amd.csr import FilterCSR
    rng = np.random.default_rng(77)
    N, R, d, B, n = 5000, 9, 64, 300, 40000
    E, Rel = random_tables(rng, N, R, d)
    t = np.stack([rng.integers(0, 60, n), rng.integers(0, R, n), rng.integers(0, N, n)], axis=1)
    host = FilterCSR.from_triples(t, R).to("cuda")
    gpu = FilterCSR.from_triples_gpu(torch.from_numpy(t).cuda(), N, R)
    hr = torch.from_numpy(np.ascontiguousarray(t[:B, :2])).cuda()
    tgt = torch.from_numpy(np.ascontiguousarray(t[:B, 2])).cuda()
    Eg, Rg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel))
    Q, bias = ops.build_query("DistMult", Eg, Rg, hr)
    a = ops.rank_filtered(Q, bias, Eg, None, tgt, host.rows_for(hr), host.row_ptr, host.col)
    b = ops.rank_filtered(Q, bias, Eg, None, tgt, gpu.rows_for(hr), gpu.row_ptr, gpu.col)
    for key in a:
        assert torch.equal(a[key], b[key])


# ---------------------------------------------------------------------------------------------
# head direction: Q'(r, t) with score(x, r, t) = Q' . E[x]
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("model,d,kw", MODEL_CASES)
def test_build_query_head_fp32(ops, model, d, kw):
    rng = np.random.default_rng(200 + d)
    N, R, B = 300, 17, 77
    E, Rel = random_tables(rng, N, R, d, std=0.5)
    rt = np.stack([rng.integers(0, R, B), rng.integers(0, N, B)], axis=1).astype(np.int64)
    Q, bias = ops.build_query(model, dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)),
                              dev(torch.from_numpy(rt)), head=True, **_gpu_kwargs(kw))
    Qr = ko.head_query(model, E, Rel, rt, **kw)
    ok, worst = score_close(Q.cpu().numpy(), Qr, 1e-5)
    assert ok, worst
    assert float(bias.abs().max()) == 0.0
    # one triple, both directions, through the library: S_tail[b, t] == S_head[b, h]
    h = rng.integers(0, N, B).astype(np.int64)
    hr = np.stack([h, rt[:, 0]], axis=1)
    Eg = dev(torch.from_numpy(E))
    Qt, bt = ops.build_query(model, Eg, dev(torch.from_numpy(Rel)), dev(torch.from_numpy(hr)), **_gpu_kwargs(kw))
    St = ops.scores(Qt, bt, Eg).cpu().numpy()[np.arange(B), rt[:, 1]]
    Sh = ops.scores(Q, bias, Eg).cpu().numpy()[np.arange(B), h]
    ref = ko.triple_scores(model, E, Rel, np.stack([h, rt[:, 0], rt[:, 1]], axis=1), **kw)
    scale = np.sqrt((ref ** 2).mean())
    assert np.abs(St - ref).max() <= 2e-5 * scale and np.abs(Sh - ref).max() <= 2e-5 * scale


@pytest.mark.parametrize("storage", ["bf16", "int8"])
@pytest.mark.parametrize("model", ["DistMult", "ComplEx", "QMult"])
def test_build_query_head_quantised_tables(ops, model, storage):
    rng = np.random.default_rng(17)
    N, R, d, B = 200, 9, 128, 50
    E, Rel = random_tables(rng, N, R, d)
    rt = np.stack([rng.integers(0, R, B), rng.integers(0, N, B)], axis=1).astype(np.int64)
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Q, _ = ops.build_query(model, dev(Et), dev(Rt), dev(torch.from_numpy(rt)), ent_scale=dev(sc), head=True)
    ok, worst = score_close(Q.cpu().numpy(), ko.head_query(model, Ev, Rv, rt), 1e-5)
    assert ok, worst


def test_build_query_head_argument_checks(ops):
    from dicee_amd._lib import KgeError
    rng = np.random.default_rng(19)
    E, Rel = random_tables(rng, 50, 4, 16)
    Eg, Rg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel))
    rt = np.array([[0, 0], [4, 1], [3, 50], [0, -1], [3, 49]], dtype=np.int64)       # (relation, tail)
    Q, bias = ops.build_query("ComplEx", Eg, Rg, dev(torch.from_numpy(rt)), head=True)
    Q = Q.cpu().numpy()
    assert np.isnan(Q[1]).all() and np.isnan(Q[2]).all() and np.isnan(Q[3]).all()
    assert np.isfinite(Q[0]).all() and np.isfinite(Q[4]).all()
    ones = torch.ones(16, device="cuda")
    norm = {"kind": "LayerNorm", "eps": 1e-5, "h_a": ones, "h_b": ones, "r_a": ones, "r_b": ones}
    with pytest.raises(KgeError) as err:
        ops.build_query("ComplEx", Eg, Rg, dev(torch.from_numpy(rt)), head=True, norm=norm)
    assert err.value.code == 2


# ---------------------------------------------------------------------------------------------
# backward of the query builder
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("model,d,kw", MODEL_CASES)
def test_build_query_backward_fp32(ops, model, d, kw):
    """d_ent / d_rel / d_coeff against central differences of the oracle's query builder (fp64).  Pairs share
    heads and relations (17 relations, 77 pairs), so the scatter with atomics is exercised too."""
    rng = np.random.default_rng(300 + d)
    N, R, B = 60, 17, 77
    E, Rel = random_tables(rng, N, R, d, std=0.5)
    hr = random_hr(rng, N, R, B)
    dQ = rng.standard_normal((B, d)).astype(np.float32)
    dbias = rng.standard_normal(B).astype(np.float32)
    Eg, Rg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel))
    d_ent = torch.zeros_like(Eg)
    d_rel = torch.zeros_like(Rg)
    gkw = _gpu_kwargs(kw)
    dcoeff = ops.build_query_backward(model, Eg, Rg, dev(torch.from_numpy(hr)), dev(torch.from_numpy(dQ)),
                                      dev(torch.from_numpy(dbias)), d_ent, d_rel, **gkw)
    wE, wR, wc = ko.build_query_backward(model, E, Rel, hr, dQ, dbias, **kw)
    for got, want, name in ((d_ent, wE, "d_ent"), (d_rel, wR, "d_rel")):
        got = got.cpu().numpy()
        rms = np.sqrt((want ** 2).mean())
        assert np.abs(got - want).max() <= 2e-5 * rms + 1e-6, (name, np.abs(got - want).max() / rms)
    for got, key in zip(dcoeff, ("coeff_p", "coeff_q", "coeff_r")):
        if key in wc:
            want = wc[key]
            assert np.abs(got.cpu().numpy() - want).max() <= 2e-5 * np.abs(want).max() + 1e-4, key
        else:
            assert got is None or kw.get(key) is not None


_NORM_BWD_CASES = [
    ("DistMult", 32, {}),
    ("ComplEx", 24, {}),
    ("QMult", 32, {}),                                # LayerNorm, then the quaternion normaliser on top of it
    ("QMult", 72, {"normalize_relation": False}),     # what the model classes run (quaternion.py:138)
    ("OMult", 24, {}),
    ("Keci", 28, {"p": 1, "q": 2, "coeff_p": [0.7], "coeff_q": [1.3, -0.4]}),
    ("DeCaL", 28, {"p": 2, "q": 2, "r": 2, "coeff_p": [0.7, 1.1], "coeff_q": [1.3, -0.4], "coeff_r": [0.6, 1.2]}),
]


@pytest.mark.parametrize("kind", ["LayerNorm", "BatchNorm1d"])
@pytest.mark.parametrize("model,d,kw", _NORM_BWD_CASES)
def test_build_query_backward_through_the_normalisation_layer(ops, model, d, kw, kind):
    """d_ent / d_rel / d_coeff and LayerNorm's own parameter gradients against central differences of the oracle's
    query builder with the same layer (fp64); BatchNorm1d with its running statistics."""
    rng = np.random.default_rng(700 + d)
    N, R, B = 40, 9, 53
    E, Rel = random_tables(rng, N, R, d, std=0.8)
    hr = random_hr(rng, N, R, B)
    dQ = rng.standard_normal((B, d)).astype(np.float32)
    dbias = rng.standard_normal(B).astype(np.float32)
    if kind == "LayerNorm":
        a_h, a_r = rng.uniform(0.5, 1.5, d).astype(np.float32), rng.uniform(-1.5, 1.5, d).astype(np.float32)
        b_h, b_r = rng.normal(0, 0.3, d).astype(np.float32), rng.normal(0, 0.3, d).astype(np.float32)
        onorm = {"kind": kind, "h_weight": a_h, "h_bias": b_h, "r_weight": a_r, "r_bias": b_r}
    else:
        a_h, a_r = rng.normal(0, 0.3, d).astype(np.float32), rng.normal(0, 0.3, d).astype(np.float32)
        b_h, b_r = rng.uniform(0.5, 2, d).astype(np.float32), rng.uniform(0.5, 2, d).astype(np.float32)
        onorm = {"kind": kind, "h_mean": a_h, "h_var": b_h, "r_mean": a_r, "r_var": b_r}
    gnorm = {"kind": kind, "eps": 1e-5, "h_a": dev(torch.from_numpy(a_h)), "h_b": dev(torch.from_numpy(b_h)),
             "r_a": dev(torch.from_numpy(a_r)), "r_b": dev(torch.from_numpy(b_r))}
    Eg, Rg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel))
    d_ent, d_rel = torch.zeros_like(Eg), torch.zeros_like(Rg)
    dnorm = {k: torch.zeros(d, device="cuda") for k in ("h_a", "h_b", "r_a", "r_b")} if kind == "LayerNorm" else None
    dcoeff = ops.build_query_backward(model, Eg, Rg, dev(torch.from_numpy(hr)), dev(torch.from_numpy(dQ)),
                                      dev(torch.from_numpy(dbias)), d_ent, d_rel, norm=gnorm, dnorm=dnorm,
                                      **_gpu_kwargs(kw))
    wE, wR, wc = ko.build_query_backward(model, E, Rel, hr, dQ, dbias, norm=onorm, **kw)
    for got, want, name in ((d_ent, wE, "d_ent"), (d_rel, wR, "d_rel")):
        got = got.cpu().numpy()
        rms = np.sqrt((want ** 2).mean())
        assert np.abs(got - want).max() <= 5e-5 * rms + 2e-6, (name, np.abs(got - want).max() / rms)
    for got, key in zip(dcoeff, ("coeff_p", "coeff_q", "coeff_r")):
        if key in wc:
            assert np.abs(got.cpu().numpy() - wc[key]).max() <= 5e-5 * np.abs(wc[key]).max() + 1e-4, key
    if kind == "LayerNorm":
        for gk, ok_ in (("h_a", "h_weight"), ("h_b", "h_bias"), ("r_a", "r_weight"), ("r_b", "r_bias")):
            want = wc[ok_]
            got = dnorm[gk].cpu().numpy()
            assert np.abs(got - want).max() <= 5e-5 * np.sqrt((want ** 2).mean()) + 1e-5, (gk, got[:4], want[:4])


@pytest.mark.parametrize("model,d,kw,B", [("DistMult", 16, {}, 12), ("ComplEx", 70, {}, 9), ("QMult", 16, {}, 11),
                                          ("Keci", 15, {"p": 2, "q": 2, "coeff_p": [0.7, 1.1], "coeff_q": [1.3, -0.4]}, 10),
                                          ("OMult", 16, {"normalize_relation": False}, 2)])
def test_batchnorm_training_mode_statistics_forward_and_backward(ops, model, d, kw, B):
    """BatchNorm1d(affine=False) with the statistics of the batch: the statistics and the running-statistics update
    against the oracle, the query vectors built with them, and the gradient through them against central
    differences of the whole batch (fp64).  Pairs repeat heads and relations."""
    rng = np.random.default_rng(900 + d)
    N, R = 7, 3
    E, Rel = random_tables(rng, N, R, d, std=0.8)
    hr = random_hr(rng, N, R, B)
    dQ = rng.standard_normal((B, d)).astype(np.float32)
    dbias = rng.standard_normal(B).astype(np.float32)
    run0 = {"h_mean": rng.normal(0, 0.2, d), "h_var": rng.uniform(0.5, 2, d), "r_mean": rng.normal(0, 0.2, d),
            "r_var": rng.uniform(0.5, 2, d)}
    running = {k: dev(torch.from_numpy(v.astype(np.float32))) for k, v in run0.items()}
    Eg, Rg, hrg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)), dev(torch.from_numpy(hr))
    norm = ops.batchnorm_stats(Eg, Rg, hrg, eps=1e-5, momentum=0.1, running=running)
    rows = {"h": E[hr[:, 0]].astype(np.float64), "r": Rel[hr[:, 1]].astype(np.float64)}
    for side in "hr":
        x = rows[side]
        np.testing.assert_allclose(norm[side + "_a"].cpu().numpy(), x.mean(axis=0), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(norm[side + "_b"].cpu().numpy(), x.var(axis=0), rtol=1e-5, atol=1e-7)
        rm, rv = ko.batch_norm_running_update(x, run0[side + "_mean"].astype(np.float32), run0[side + "_var"].astype(np.float32), 0.1)
        np.testing.assert_allclose(running[side + "_mean"].cpu().numpy(), rm, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(running[side + "_var"].cpu().numpy(), rv, rtol=1e-5, atol=1e-7)
    onorm = {"kind": "BatchNorm1dTrain", "eps": 1e-5}
    gkw = _gpu_kwargs(kw)
    Q, bias = ops.build_query(model, Eg, Rg, hrg, norm=norm, **gkw)
    Qr, br = ko.build_query(model, E, Rel, hr, norm=onorm, **kw)
    ok, worst = score_close(Q.cpu().numpy(), Qr, 5e-5)
    assert ok, worst
    d_ent, d_rel = torch.zeros_like(Eg), torch.zeros_like(Rg)
    ops.build_query_backward(model, Eg, Rg, hrg, dev(torch.from_numpy(dQ)), dev(torch.from_numpy(dbias)), d_ent, d_rel,
                             norm=norm, **gkw)
    wE, wR = ko.build_query_backward_batch(model, E, Rel, hr, dQ, dbias, norm=onorm, **kw)
    for got, want, name in ((d_ent, wE, "d_ent"), (d_rel, wR, "d_rel")):
        got = got.cpu().numpy()
        rms = np.sqrt((want ** 2).mean())
        assert np.abs(got - want).max() <= 2e-4 * rms + 2e-5, (name, np.abs(got - want).max() / rms)


def test_batchnorm_statistics_over_a_large_batch_and_bad_arguments(ops):
    from dicee_amd._lib import KgeError
    rng = np.random.default_rng(77)
    N, R, d, B = 500, 11, 200, 5000          # several batch slices per feature block, a ragged last feature block
    E, Rel = random_tables(rng, N, R, d, std=1.0)
    E += 3.0                                 # a mean far from zero: the variance must not cancel
    hr = random_hr(rng, N, R, B)
    Eg, Rg, hrg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)), dev(torch.from_numpy(hr))
    norm = ops.batchnorm_stats(Eg, Rg, hrg)
    x, y = E[hr[:, 0]].astype(np.float64), Rel[hr[:, 1]].astype(np.float64)
    np.testing.assert_allclose(norm["h_a"].cpu().numpy(), x.mean(axis=0), rtol=1e-6)
    np.testing.assert_allclose(norm["h_b"].cpu().numpy(), x.var(axis=0), rtol=1e-5)
    np.testing.assert_allclose(norm["r_b"].cpu().numpy(), y.var(axis=0), rtol=1e-5)
    with pytest.raises(ValueError):          # torch: "Expected more than 1 value per channel when training"
        ops.batchnorm_stats(Eg, Rg, hrg[:1].contiguous())
    bad = hr.copy()
    bad[17, 0] = N
    nb = ops.batchnorm_stats(Eg, Rg, dev(torch.from_numpy(bad)))
    assert torch.isnan(nb["h_a"]).all() and torch.isnan(nb["r_b"]).all()
    with pytest.raises(KgeError):            # the backward needs the statistics of at least two rows as well
        ops.build_query_backward("DistMult", Eg, Rg, hrg[:1].contiguous(), torch.ones(1, d, device="cuda"), None,
                                 torch.zeros_like(Eg), torch.zeros_like(Rg), norm=norm)


@pytest.mark.parametrize("layer", ["none", "LayerNorm", "BatchNorm1d", "BatchNorm1dTrain"])
@pytest.mark.parametrize("model,d,kw", [("DistMult", 24, {}), ("QMult", 16, {}), ("ComplEx", 70, {}),
                                        ("Keci", 15, {"p": 2, "q": 2, "coeff_p": [0.7, 1.1], "coeff_q": [1.3, -0.4]})])
def test_dropout_masks_forward_and_backward(ops, model, d, kw, layer):
    """Training-mode dropout with the caller's masks on the looked-up rows (and on DistMult's h * r), alone and in
    front of each normalisation layer: query vectors and gradients against the oracle with the same masks."""
    rng = np.random.default_rng(1100 + d)
    N, R, B = 9, 4, 13
    E, Rel = random_tables(rng, N, R, d, std=0.8)
    hr = random_hr(rng, N, R, B)
    dQ = rng.standard_normal((B, d)).astype(np.float32)
    dbias = rng.standard_normal(B).astype(np.float32)
    keep = {k: (rng.random((B, d)) >= 0.3).astype(np.uint8) for k in ("keep_h", "keep_r")}
    if model == "DistMult":
        keep["keep_q"] = (rng.random((B, d)) >= 0.4).astype(np.uint8)
    odrop = dict(keep, scale_in=1 / 0.7, scale_hidden=1 / 0.6)
    gdrop = {k: (dev(torch.from_numpy(v)) if k.startswith("keep") else v) for k, v in odrop.items()}
    Eg, Rg, hrg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)), dev(torch.from_numpy(hr))
    onorm = gnorm = dnorm = None
    if layer == "LayerNorm":
        a_h, a_r = rng.uniform(0.5, 1.5, d).astype(np.float32), rng.uniform(0.5, 1.5, d).astype(np.float32)
        b_h, b_r = rng.normal(0, 0.3, d).astype(np.float32), rng.normal(0, 0.3, d).astype(np.float32)
        onorm = {"kind": layer, "h_weight": a_h, "h_bias": b_h, "r_weight": a_r, "r_bias": b_r}
        dnorm = {k: torch.zeros(d, device="cuda") for k in ("h_a", "h_b", "r_a", "r_b")}
    elif layer == "BatchNorm1d":
        a_h, a_r = rng.normal(0, 0.3, d).astype(np.float32), rng.normal(0, 0.3, d).astype(np.float32)
        b_h, b_r = rng.uniform(0.5, 2, d).astype(np.float32), rng.uniform(0.5, 2, d).astype(np.float32)
        onorm = {"kind": layer, "h_mean": a_h, "h_var": b_h, "r_mean": a_r, "r_var": b_r}
    if layer in ("LayerNorm", "BatchNorm1d"):
        gnorm = {"kind": layer, "eps": 1e-5, "h_a": dev(torch.from_numpy(a_h)), "h_b": dev(torch.from_numpy(b_h)),
                 "r_a": dev(torch.from_numpy(a_r)), "r_b": dev(torch.from_numpy(b_r))}
    elif layer == "BatchNorm1dTrain":
        onorm = {"kind": layer, "eps": 1e-5}
        gnorm = ops.batchnorm_stats(Eg, Rg, hrg, dropout=gdrop)
        x = E[hr[:, 0]].astype(np.float64) * keep["keep_h"] * (1 / 0.7)
        np.testing.assert_allclose(gnorm["h_a"].cpu().numpy(), x.mean(axis=0), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(gnorm["h_b"].cpu().numpy(), x.var(axis=0), rtol=1e-5, atol=1e-6)
    gkw = _gpu_kwargs(kw)
    Q, bias = ops.build_query(model, Eg, Rg, hrg, norm=gnorm, dropout=gdrop, **gkw)
    Qr, br = ko.build_query(model, E, Rel, hr, norm=onorm, dropout=odrop, **kw)
    ok, worst = score_close(Q.cpu().numpy(), Qr, 5e-5)
    assert ok, worst
    assert np.abs(bias.cpu().numpy() - br).max() <= 5e-5 * (np.abs(br).max() + 1)
    d_ent, d_rel = torch.zeros_like(Eg), torch.zeros_like(Rg)
    ops.build_query_backward(model, Eg, Rg, hrg, dev(torch.from_numpy(dQ)), dev(torch.from_numpy(dbias)), d_ent, d_rel,
                             norm=gnorm, dnorm=dnorm, dropout=gdrop, **gkw)
    if layer == "BatchNorm1dTrain":
        wE, wR = ko.build_query_backward_batch(model, E, Rel, hr, dQ, dbias, norm=onorm, dropout=odrop, **kw)
        wc = {}
    else:
        wE, wR, wc = ko.build_query_backward(model, E, Rel, hr, dQ, dbias, norm=onorm, dropout=odrop, **kw)
    for got, want, name in ((d_ent, wE, "d_ent"), (d_rel, wR, "d_rel")):
        got = got.cpu().numpy()
        rms = np.sqrt((want ** 2).mean())
        assert np.abs(got - want).max() <= 2e-4 * rms + 2e-5, (name, np.abs(got - want).max() / rms)
    if layer == "LayerNorm":
        for gk, ok_ in (("h_a", "h_weight"), ("h_b", "h_bias"), ("r_a", "r_weight"), ("r_b", "r_bias")):
            want = wc[ok_]
            assert np.abs(dnorm[gk].cpu().numpy() - want).max() <= 1e-4 * np.sqrt((want ** 2).mean()) + 1e-5, gk


def test_dropout_argument_checks(ops):
    from dicee_amd._lib import KgeError
    rng = np.random.default_rng(6)
    E, Rel = random_tables(rng, 20, 3, 16)
    hr = random_hr(rng, 20, 3, 6)
    Eg, Rg, hrg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel)), dev(torch.from_numpy(hr))
    ones = torch.ones(6, 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(KgeError):      # a hidden mask for a model without hidden dropout
        ops.build_query("ComplEx", Eg, Rg, hrg, dropout={"keep_q": ones})
    with pytest.raises(KgeError):      # a scale below one is no 1 / (1 - rate)
        ops.build_query("DistMult", Eg, Rg, hrg, dropout={"keep_h": ones, "scale_in": 0.5})
    with pytest.raises(ValueError):
        ops.build_query("DistMult", Eg, Rg, hrg, dropout={"keep_h": ones}, head=True)
    with pytest.raises(TypeError):
        ops.build_query("DistMult", Eg, Rg, hrg, dropout={"keep_h": ones[:3]})
    # all-ones masks with scale one: the plain query vectors, bit for bit
    Q0, _ = ops.build_query("DistMult", Eg, Rg, hrg)
    Q1, _ = ops.build_query("DistMult", Eg, Rg, hrg, dropout={"keep_h": ones, "keep_r": ones, "keep_q": ones})
    assert torch.equal(Q0, Q1)


@pytest.mark.parametrize("d,layer", [(4096, "LayerNorm"), (8192, None), (4100, "LayerNorm")])
def test_build_query_backward_at_the_widest_rows(ops, d, layer):
    """The widest rows the backward keeps in LDS (5.25 rows per pair with a normalisation layer: d <= 4096; 3 rows
    without: d <= 8192), against torch autograd in float64; one element past the limit is refused."""
    from dicee_amd._lib import KgeError
    g = torch.Generator().manual_seed(d)
    N, R, B = 20, 3, 9
    E = dev(torch.randn(N, d, generator=g) * 0.5)
    Rel = dev(torch.randn(R, d, generator=g) * 0.5)
    hr = torch.stack([torch.randint(0, N, (B,), generator=g), torch.randint(0, R, (B,), generator=g)], 1)
    dQ = torch.randn(B, d, generator=g)
    norm = dn = None
    if layer:
        w = [torch.rand(d, generator=g) + 0.5 for _ in range(2)]
        b = [torch.randn(d, generator=g) * 0.1 for _ in range(2)]
        norm = {"kind": layer, "eps": 1e-5, "h_a": dev(w[0]), "h_b": dev(b[0]), "r_a": dev(w[1]), "r_b": dev(b[1])}
        dn = {k: torch.zeros(d, device="cuda") for k in ("h_a", "h_b", "r_a", "r_b")}
    dE, dR = torch.zeros_like(E), torch.zeros_like(Rel)
    if d > 4096 and layer:
        with pytest.raises(KgeError) as err:
            ops.build_query_backward("DistMult", E, Rel, dev(hr), dev(dQ), None, dE, dR, norm=norm, dnorm=dn)
        assert err.value.code == 2
        return
    ops.build_query_backward("DistMult", E, Rel, dev(hr), dev(dQ), None, dE, dR, norm=norm, dnorm=dn)
    Et, Rt = E.double().cpu().requires_grad_(), Rel.double().cpu().requires_grad_()
    h, r = Et[hr[:, 0]], Rt[hr[:, 1]]
    if layer:
        h = torch.nn.functional.layer_norm(h, (d,), w[0].double(), b[0].double(), 1e-5)
        r = torch.nn.functional.layer_norm(r, (d,), w[1].double(), b[1].double(), 1e-5)
    ((h * r) * dQ.double()).sum().backward()
    for got, want in ((dE, Et.grad), (dR, Rt.grad)):
        assert (got.double().cpu() - want).abs().max().item() <= 2e-5 * want.abs().max().item()


def test_build_query_backward_norm_argument_checks(ops):
    from dicee_amd._lib import KgeError
    rng = np.random.default_rng(5)
    E, Rel = random_tables(rng, 20, 3, 16)
    hr = random_hr(rng, 20, 3, 6)
    Eg, Rg = dev(torch.from_numpy(E)), dev(torch.from_numpy(Rel))
    dQ = torch.ones(6, 16, device="cuda")
    ones = torch.ones(16, device="cuda")
    bn = {"kind": "BatchNorm1d", "eps": 1e-5, "h_a": ones, "h_b": ones, "r_a": ones, "r_b": ones}
    with pytest.raises(KgeError) as err:      # BatchNorm1d(affine=False) has no parameters
        ops.build_query_backward("DistMult", Eg, Rg, dev(torch.from_numpy(hr)), dQ, None, torch.zeros_like(Eg),
                                 torch.zeros_like(Rg), norm=bn, dnorm={"h_a": torch.zeros(16, device="cuda")})
    assert err.value.code == 1
    # norm of kind none: the plain backward, bit for bit
    a, b = torch.zeros_like(Eg), torch.zeros_like(Rg)
    ops.build_query_backward("DistMult", Eg, Rg, dev(torch.from_numpy(hr)), dQ, None, a, b)
    assert float(a.abs().sum()) > 0


# ---------------------------------------------------------------------------------------------
# top-k over tables built to defeat its shortcuts: several rounds, guessed thresholds, overflowing buffers, repairs
# ---------------------------------------------------------------------------------------------
def _topk_stress_cases():
    cases = []
    i = 0
    for storage, d in (("fp32", 32), ("bf16", 128), ("bf16", 64), ("int8", 128), ("int8", 64)):
        for pattern in ("pool1", "pool3", "pool50", "ascending", "descending", "two_values", "zero_rows"):
            k = (1, 7, 100, 1000)[i % 4]
            N = (5000, 20011, 70001)[i % 3]
            B = (1, 5, 70)[(i // 2) % 3]
            cases.append((i, storage, d, pattern, N, B, k))
            i += 1
    return cases


@pytest.mark.parametrize("seed,storage,d,pattern,N,B,k", _topk_stress_cases())
def test_topk_stress_patterns_match_the_materialised_scores(ops, seed, storage, d, pattern, N, B, k):
    """Tables whose scores tie massively (rows drawn from a pool of 1, 3 or 50 distinct rows; only two distinct
    scores; thousands of all-zero rows) or arrive in the worst order (best rows last: every guessed threshold fails;
    best rows first), for every storage and across the rounds of a call: the result must be the top k of the
    library's own scores, ties towards the lower entity id."""
    rng = np.random.default_rng(1000 + seed)
    k = min(k, N)
    Q = (rng.standard_normal((B, d)) * 0.3).astype(np.float32)
    ints = rng.integers(-90, 91, (N, d)).astype(np.int8)                  # every storage holds these exactly
    if pattern.startswith("pool"):
        pool = rng.integers(-90, 91, (int(pattern[4:]), d)).astype(np.int8)
        ints = pool[rng.integers(0, len(pool), N)]
    elif pattern == "two_values":
        v = rng.integers(-90, 91, d).astype(np.int8)
        ints = np.where(rng.random(N)[:, None] < 0.5, v[None, :], -v[None, :]).astype(np.int8)
    elif pattern == "zero_rows":
        ints[rng.random(N) < 0.4] = 0
    if pattern in ("ascending", "descending"):
        s0 = ints.astype(np.float64) @ Q[0].astype(np.float64)           # order by the first query's scores
        order = np.argsort(s0 if pattern == "ascending" else -s0, kind="stable")
        ints = ints[order]
    if storage == "int8":
        E, sc = dev(torch.from_numpy(ints)), dev(torch.full((N,), 0.01))
    else:
        E, sc = dev(torch.from_numpy(ints.astype(np.float32) * 0.01)), None
        if storage == "bf16":
            E = E.to(torch.bfloat16)
    Qg = dev(torch.from_numpy(Q))
    vals, idx = ops.topk(Qg, None, E, sc, k)
    S = ops.scores(Qg, None, E, sc).cpu().numpy()
    wv, wi = ko.topk(S, k)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)


@pytest.mark.parametrize("storage,d", [("fp32", 32), ("bf16", 128), ("bf16", 64), ("int8", 128), ("int8", 64), ("bf16", 256),
                                       ("bf16", 200), ("int8", 144), ("bf16", 512), ("bf16", 360), ("int8", 512), ("int8", 368)])
@pytest.mark.parametrize("pattern", ["pool1", "pool3", "pool50", "two_values", "zero_rows"])
def test_rank_stress_patterns_match_the_materialised_scores(ops, FilterCSR, storage, d, pattern):
    """The same massively tied tables under the filtered rank: the target ties with thousands of entities (every
    stage of the bf16 d = 128 main loop takes its exact second pass), filter rows hold tied entities and the target
    itself; counters must equal those counted on the library's own scores."""
    rng = np.random.default_rng(sum(ord(ch) for ch in storage + pattern) * 1000 + d)
    N, R, B = 9001, 5, 700
    Q = (rng.standard_normal((B, d)) * 0.3).astype(np.float32)
    ints = rng.integers(-90, 91, (N, d)).astype(np.int8)
    if pattern.startswith("pool"):
        pool = rng.integers(-90, 91, (int(pattern[4:]), d)).astype(np.int8)
        ints = pool[rng.integers(0, len(pool), N)]
    elif pattern == "two_values":
        v = rng.integers(-90, 91, d).astype(np.int8)
        ints = np.where(rng.random(N)[:, None] < 0.5, v[None, :], -v[None, :]).astype(np.int8)
    elif pattern == "zero_rows":
        ints[rng.random(N) < 0.4] = 0
    if storage == "int8":
        E, sc = dev(torch.from_numpy(ints)), dev(torch.full((N,), 0.01))
    else:
        E, sc = dev(torch.from_numpy(ints.astype(np.float32) * 0.01)), None
        if storage == "bf16":
            E = E.to(torch.bfloat16)
    Qg = dev(torch.from_numpy(Q))
    bias = dev(torch.from_numpy(rng.standard_normal(B).astype(np.float32)))
    hr = random_hr(rng, N, R, B)
    hr[B // 2:] = hr[:B - B // 2]                                    # every filter row shared by two queries ...
    Q[B // 2:] = Q[:B - B // 2]                                      # ... that hold the same vector, as (h, r) pairs do
    Qg = dev(torch.from_numpy(Q))
    targets = rng.integers(0, N, B).astype(np.int64)
    er = random_csr(rng, hr, targets, N, R, max_len=40)
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    hr_g = dev(torch.from_numpy(hr))
    out = ops.rank_filtered(Qg, bias, E, sc, dev(torch.from_numpy(targets)), csr.rows_for(hr_g), csr.row_ptr, csr.col)
    S_raw = ops.scores(Qg, None, E, sc).cpu().numpy()
    g, t, tl = _expected_counts(S_raw, targets, [er[(int(h), int(r))] for h, r in hr])
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)
    if pattern == "pool1":
        assert t.max() > N // 2                                       # the ties are really there


# ---------------------------------------------------------------------------------------------
# seeded sweep over awkward shapes: every fused epilogue against the library's own materialised scores
# ---------------------------------------------------------------------------------------------
def _sweep_cases():
    rng = np.random.default_rng(2024)
    cases = []
    for i in range(36):
        storage = ("fp32", "bf16", "int8")[i % 3]
        if storage == "fp32":
            d = int(rng.choice([1, 3, 4, 8, 20, 33, 64, 100, 200]))
        elif storage == "bf16":
            d = int(rng.choice([8, 16, 40, 64, 128]))
        else:
            d = int(rng.choice([16, 32, 64, 128]))
        N = int(rng.choice([1, 2, 31, 32, 33, 127, 128, 129, 257, 1000, 1025, 4097]))
        B = int(rng.choice([1, 2, 63, 64, 65, 255, 257, 513]))
        cases.append((i, storage, d, N, B))
    # bf16 rows wider than 256 elements (the query row in registers, entity rows through LDS by segments)
    for j, (d, N, B) in enumerate([(264, 33, 1), (384, 1, 257), (392, 129, 65), (512, 4097, 513), (512, 31, 2),
                                   (456, 1025, 255), (272, 257, 64)]):
        cases.append((36 + j, "bf16", d, N, B))
    for j, (d, N, B) in enumerate([(272, 33, 1), (384, 1, 257), (400, 129, 65), (512, 4097, 513), (512, 31, 2),
                                   (464, 1025, 255)]):
        cases.append((43 + j, "int8", d, N, B))
    return cases


@pytest.mark.parametrize("seed,storage,d,N,B", _sweep_cases())
def test_shape_sweep_all_epilogues_agree_with_materialised_scores(ops, FilterCSR, seed, storage, d, N, B):
    rng = np.random.default_rng(seed)
    R = 3
    E, Rel = random_tables(rng, N, R, d)
    if N >= 3:
        E[N - 1] = E[0]                                               # an exact tie at the table's last row
    hr = random_hr(rng, N, R, B)
    Et, sc, Rt, Ev, Rv = stored_tables(E, Rel, storage)
    Eg, scg = dev(Et), dev(sc)
    hr_g = dev(torch.from_numpy(hr))
    Q, bias = ops.build_query("DistMult", Eg, dev(Rt), hr_g, ent_scale=scg)
    S = ops.scores(Q, bias, Eg, scg)
    assert S.shape == (B, N)
    S_raw = ops.scores(Q, None, Eg, scg).cpu().numpy()
    ref = ko.k_vs_all_scores("DistMult", Ev, Rv, hr)
    # with a handful of entities a row has no typical score size to measure against: bound the error by the
    # sizes of the two vectors instead (rounding both to bf16 perturbs a dot product by < 2^-8 |q| |e|)
    qn = np.linalg.norm(Ev[hr[:, 0]] * Rv[hr[:, 1]], axis=1)[:, None] * np.linalg.norm(Ev, axis=1)[None, :]
    assert np.all(np.abs(S.cpu().numpy() - ref) <= RTOL[storage] * np.maximum(qn, np.abs(ref)) + 1e-30)
    # filtered rank
    targets = rng.integers(0, N, B).astype(np.int64)
    er = random_csr(rng, hr, targets, N, R, max_len=min(6, N))
    csr = FilterCSR.from_er_vocab(er, R, device="cuda")
    out = ops.rank_filtered(Q, bias, Eg, scg, dev(torch.from_numpy(targets)), csr.rows_for(hr_g), csr.row_ptr, csr.col)
    g, t, tl = _expected_counts(S_raw, targets, [er[(int(h), int(r))] for h, r in hr])
    np.testing.assert_array_equal(out["n_greater"].cpu().numpy(), g)
    np.testing.assert_array_equal(out["n_equal"].cpu().numpy(), t)
    np.testing.assert_array_equal(out["n_equal_lower"].cpu().numpy(), tl)
    # top-k, k up to N
    k = int(min(N, rng.choice([1, 2, 10, 100])))
    vals, idx = ops.topk(Q, bias, Eg, scg, k)
    wv, wi = ko.topk(S.cpu().numpy(), k)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)
    np.testing.assert_array_equal(vals.cpu().numpy(), wv)
    # row extrema and one given entity per query
    lo, hi = ops.row_minmax(Q, bias, Eg, scg)
    np.testing.assert_array_equal(lo.cpu().numpy(), S.cpu().numpy().min(1))
    np.testing.assert_array_equal(hi.cpu().numpy(), S.cpu().numpy().max(1))
    one = ops.triple_scores(Q, bias, Eg, scg, dev(torch.from_numpy(targets)))
    np.testing.assert_array_equal(one.cpu().numpy(), S.cpu().numpy()[np.arange(B), targets])
    # BCE against the dense closed form on the library's scores (fp64 sum)
    pos = [sorted(set(er[(int(h), int(r))])) for h, r in hr]
    loss = ops.bce_multihot(Q, bias, Eg, scg, csr.rows_for(hr_g), csr.row_ptr, csr.col, 0.0)[0].item()
    want = ko.bce_multihot(S.cpu().numpy().astype(np.float64), pos)
    assert loss == pytest.approx(want, rel=1e-4, abs=1e-6)


# ---------------------------------------------------------------------------------------------
# random differential sweep: shapes, storages, table patterns, bias on and off, filter rows shared by queries
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", list(range(8)))
def test_random_differential_sweep(ops, FilterCSR, seed):
    """Thirty random cases per seed.  Filtered-rank counters, top-k (also through a prepared int8 table), row extrema
    and single-entity scores must equal what follows from the library's own materialised scores, bit for bit: the
    counters and the top-k order from the scores before the bias, ties towards the lower entity id.  Tables of
    random rows, of small-integer rows (exact arithmetic: masses of ties), of rows drawn from a pool of one to 17,
    and half-zero tables; queries that share a filter row and a vector; with and without a per-query bias."""
    rng = np.random.default_rng(7000 + seed)
    gen = torch.Generator(device="cuda").manual_seed(7000 + seed)
    for case in range(30):
        storage = ("fp32", "bf16", "int8")[case % 3]
        B = int(rng.choice([1, 2, 31, 33, 64, 100, 257, 1000, 2500, 4097, 8193]))
        if storage == "fp32":
            d = int(rng.choice([1, 2, 5, 8, 16, 31, 32, 48, 64, 100, 128, 200, 256, 260]))
        elif storage == "bf16":
            d = int(rng.choice([8, 16, 40, 64, 72, 128, 136, 200, 248, 256, 384]))
        else:
            d = int(rng.choice([16, 32, 64, 128, 128, 128, 144, 192, 240, 256, 272]))
        N = int(rng.choice([1, 7, 64, 65, 1000, 4097, 20000, 70001] + ([150001] if case % 10 == 9 else [])))
        if B * N > 1e8:
            B = max(1, int(1e8 // N))
        pattern = str(rng.choice(["randn", "randn", "ints", "pool", "half_zero"]))
        with_bias = bool(rng.random() < 0.5)
        label = f"seed {seed} case {case}: {storage} B={B} N={N} d={d} {pattern} bias={with_bias}"
        print(label, flush=True)
        if pattern == "ints":
            E = torch.randint(-5, 6, (N, d), device="cuda", generator=gen).float() * 0.125
            Q = torch.randint(-4, 5, (B, d), device="cuda", generator=gen).float() * 0.25
        else:
            Q = torch.randn(B, d, device="cuda", generator=gen) * 0.3
            if pattern == "pool":
                pool = torch.randn(int(rng.choice([1, 2, 17])), d, device="cuda", generator=gen)
                E = pool[torch.randint(0, pool.shape[0], (N,), device="cuda", generator=gen)]
            else:
                E = torch.randn(N, d, device="cuda", generator=gen) * 0.3
                if pattern == "half_zero":
                    E[torch.rand(N, device="cuda", generator=gen) < 0.5] = 0
        bias = torch.randn(B, device="cuda", generator=gen) if with_bias else None
        sc = None
        if storage == "bf16":
            Et = E.to(torch.bfloat16).contiguous()
        elif storage == "int8":
            sc = (E.abs().amax(1) / 127).clamp_min(1e-12)
            Et = torch.round(E / sc[:, None]).clamp(-127, 127).to(torch.int8).contiguous()
            if rng.random() < 0.3:
                sc = sc * torch.exp(torch.randn(N, device="cuda", generator=gen) * 2)
        else:
            Et = E.contiguous()
        del E
        R = 3
        hr = torch.stack([torch.randint(0, N, (B,), device="cuda", generator=gen),
                          torch.randint(0, R, (B,), device="cuda", generator=gen)], 1)
        if rng.random() < 0.5 and B > 4:                                  # pairs of queries with one row and one vector
            hr[B // 2:] = hr[:B - B // 2].clone()
            Q[B // 2:] = Q[:B - B // 2].clone()
        S_raw = ops.scores(Q, None, Et, sc)
        S = ops.scores(Q, bias, Et, sc) if with_bias else S_raw
        rows_all = torch.arange(B, device="cuda")
        tgt = torch.randint(0, N, (B,), device="cuda", generator=gen)
        # ---- filtered rank ----
        per_query = int(rng.choice([0, 1, 5, 40]))
        mask = torch.zeros((B, N), dtype=torch.bool, device="cuda")
        if per_query == 0:
            out = ops.rank_filtered(Q, bias, Et, sc, tgt)
        else:
            T = min(200000, B * per_query)
            qi = torch.randint(0, B, (T,), device="cuda", generator=gen)
            tails = torch.randint(0, N, (T,), device="cuda", generator=gen)
            triples = torch.stack([hr[qi, 0], hr[qi, 1], tails], 1)
            csr = FilterCSR.from_triples(triples.cpu().numpy(), R, device="cuda")
            out = ops.rank_filtered(Q, bias, Et, sc, tgt, csr.rows_for(hr), csr.row_ptr, csr.col)
            # every query whose (head, relation) pair equals the triple's is filtered by it
            key_q = hr[:, 0] * R + hr[:, 1]
            key_t = triples[:, 0] * R + triples[:, 1]
            order = torch.argsort(key_q)
            ks = key_q[order]
            lo = torch.searchsorted(ks, key_t, right=False)
            hi = torch.searchsorted(ks, key_t, right=True)
            reps = hi - lo
            t_idx = torch.repeat_interleave(torch.arange(T, device="cuda"), reps)
            offs = torch.arange(int(reps.sum()), device="cuda") - torch.repeat_interleave(torch.cumsum(reps, 0) - reps, reps)
            mask[order[lo[t_idx] + offs], tails[t_idx]] = True
        mask[rows_all, tgt] = False                                      # the target itself always counts
        thr = S_raw[rows_all, tgt][:, None]
        keep = ~mask
        eq = (S_raw == thr) & keep
        assert torch.equal(out["n_greater"], ((S_raw > thr) & keep).sum(1).int()), label
        assert torch.equal(out["n_equal"], eq.sum(1).int() - 1), label
        assert torch.equal(out["n_equal_lower"], (eq & (torch.arange(N, device="cuda")[None, :] < tgt[:, None])).sum(1).int()), label
        del mask, keep, eq
        # ---- top-k ----
        k = min(N, int(rng.choice([1, 3, 10, 100, 500, 1024])))
        vals, idx = ops.topk(Q, bias, Et, sc, k)
        key = S_raw.clone()
        tv, ti = torch.sort(key, dim=1, descending=True, stable=True)
        tv, ti = tv[:, :k], ti[:, :k]
        if with_bias:
            tv = tv + bias[:, None]
        assert torch.equal(vals, tv), label
        differ = idx != ti
        assert bool((tv[differ] == (bias[:, None].expand_as(tv)[differ] if with_bias else 0)).all()), label  # -0 / +0 only
        if storage == "int8" and d == 128:
            v2, i2 = ops.topk(Q, bias, Et, sc, k, prepared=ops.topk_prepare(Et, sc))
            assert torch.equal(v2, vals) and torch.equal(i2, idx), label
        # ---- extrema, one entity per query ----
        lo_, hi_ = ops.row_minmax(Q, bias, Et, sc)
        assert torch.equal(lo_, S.min(1).values) and torch.equal(hi_, S.max(1).values), label
        assert torch.equal(ops.triple_scores(Q, bias, Et, sc, tgt), S[rows_all, tgt]), label
        del S, S_raw, key, tv, ti
