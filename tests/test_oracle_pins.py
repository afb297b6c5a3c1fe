"""Independent checks that pin the CPU oracle (no GPU, no reference import).

Each test compares an oracle function with something that does not share its
formula: a brute-force loop, a textbook/library routine, a different algebraic
representation (complex128, a structure-constant table, a bitmask geometric
algebra), a hand-computed fixture under ``tests/golden``, or an invariant.
"""
import itertools
import json
import os

import numpy as np
import pytest
import torch

from oracle import kge_oracle as ko
from oracle import torch_cpu_path as tcp

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _tables(rng, N, R, d, sd=0.1):
    return rng.normal(0, sd, (N, d)), rng.normal(0, sd, (R, d))


def _hr(rng, N, R, B):
    return np.stack([rng.integers(0, N, B), rng.integers(0, R, B)], axis=1)


# ------------------------------------------------------------------ DistMult
def test_distmult_bruteforce():
    rng = np.random.default_rng(0)
    E, R = _tables(rng, 7, 3, 6)
    hr = _hr(rng, 7, 3, 5)
    S = ko.k_vs_all_scores("DistMult", E, R, hr)
    for b, (h, r) in enumerate(hr):
        for e in range(7):
            acc = 0.0
            for k in range(6):
                acc += E[h, k] * R[r, k] * E[e, k]
            assert S[b, e] == pytest.approx(acc, rel=1e-12, abs=1e-15)


# ------------------------------------------------------------------- ComplEx
def test_complex_vs_complex128_hermitian_product():
    rng = np.random.default_rng(1)
    N, Rn, d = 11, 4, 10
    E, R = _tables(rng, N, Rn, d)
    hr = _hr(rng, N, Rn, 6)
    S = ko.k_vs_all_scores("ComplEx", E, R, hr)
    Ec = E[:, :d // 2] + 1j * E[:, d // 2:]
    Rc = R[:, :d // 2] + 1j * R[:, d // 2:]
    ref = np.real((Ec[hr[:, 0]] * Rc[hr[:, 1]]) @ np.conj(Ec).T)
    np.testing.assert_allclose(S, ref, rtol=1e-12, atol=1e-15)
    # the reference's 4-mm decomposition agrees with the single-GEMM form
    np.testing.assert_allclose(ko.k_vs_all_scores_ref_form("ComplEx", E, R, hr), S, rtol=1e-12, atol=1e-15)


def test_complex_sign_of_each_term():
    # one-hot probes: a wrong sign or swapped half flips exactly one of these
    d = 2
    E = np.array([[1.0, 0.0], [0.0, 1.0]])      # e0 = 1, e1 = i
    R = np.array([[1.0, 0.0], [0.0, 1.0]])      # r0 = 1, r1 = i
    hr = np.array([[0, 0], [0, 1], [1, 0], [1, 1]])
    S = ko.k_vs_all_scores("ComplEx", E, R, hr)
    # Re(h r conj(t)):  (1*1)->[1,0]; (1*i)=i->[0,1]; (i*1)=i->[0,1]; (i*i)=-1->[-1,0]
    np.testing.assert_array_equal(S, np.array([[1, 0], [0, 1], [0, 1], [-1, 0]], dtype=float))


# --------------------------------------------------------------------- QMult
def _structure_constants():
    """T[i,j,k] with e_i e_j = sum_k T[i,j,k] e_k for (1,i,j,k), built from the
    defining relations i^2=j^2=k^2=ijk=-1 by closure, not from the product formula."""
    T = np.zeros((4, 4, 4))
    for a in range(4):
        T[0, a, a] = 1
        T[a, 0, a] = 1
    for a in (1, 2, 3):
        T[a, a, 0] = -1
    for a, b, c in ((1, 2, 3), (2, 3, 1), (3, 1, 2)):   # ij=k, jk=i, ki=j
        T[a, b, c] = 1
        T[b, a, c] = -1
    return T


def test_hamilton_product_vs_structure_constants_and_scipy():
    from scipy.spatial.transform import Rotation
    rng = np.random.default_rng(2)
    B, d4 = 5, 3
    h = rng.normal(size=(B, 4 * d4))
    r = rng.normal(size=(B, 4 * d4))
    parts = ko.hamilton_product_blocks(h, r)
    T = _structure_constants()
    hq = h.reshape(B, 4, d4)
    rq = r.reshape(B, 4, d4)
    ref = np.einsum("bin,bjn,ijk->bkn", hq, rq, T)
    for k in range(4):
        np.testing.assert_allclose(parts[k], ref[:, k, :], rtol=1e-12, atol=1e-14)
    # library cross-check on unit quaternions (scipy stores scalar last)
    a = rng.normal(size=4)
    a /= np.linalg.norm(a)
    b = rng.normal(size=4)
    b /= np.linalg.norm(b)
    prod = (Rotation.from_quat(np.r_[a[1:], a[0]]) * Rotation.from_quat(np.r_[b[1:], b[0]])).as_quat()
    mine = np.array([p[0, 0] for p in ko.hamilton_product_blocks(a[None, :], b[None, :])])
    mine_sl = np.r_[mine[1:], mine[0]]
    assert np.allclose(mine_sl, prod, atol=1e-12) or np.allclose(mine_sl, -prod, atol=1e-12)


def test_quaternion_normalizer_groups_and_eps():
    rng = np.random.default_rng(3)
    x = rng.normal(size=(4, 16))
    x[0, 4:8] = 0.0
    y = ko.quaternion_normalize(x)
    norms = np.linalg.norm(y.reshape(4, 4, 4), axis=-1)
    np.testing.assert_allclose(norms[1:], 1.0, rtol=1e-12)
    assert norms[0, 1] == 0.0 and np.all(y[0, 4:8] == 0.0)
    # library routine
    ref = torch.nn.functional.normalize(torch.tensor(x).view(4, 4, 4), p=2, dim=-1).view(4, 16).numpy()
    np.testing.assert_allclose(y, ref, rtol=1e-12, atol=0)


def test_qmult_block_vs_consecutive_quirk_fixture():
    """d=8: normalisation groups are (0..3),(4..7) but the Hamilton product pairs
    elements (g, g+2, g+4, g+6).  Expected values were computed by hand."""
    with open(os.path.join(GOLD, "qmult_d8_quirk.json")) as f:
        fx = json.load(f)
    E = np.array(fx["E"])
    R = np.array(fx["R"])
    hr = np.array(fx["hr"])
    S = ko.k_vs_all_scores("QMult", E, R, hr)
    np.testing.assert_allclose(S, np.array(fx["scores"]), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(ko.k_vs_all_scores_ref_form("QMult", E, R, hr), S, rtol=1e-12, atol=1e-14)


def test_qmult_single_gemm_identity():
    rng = np.random.default_rng(4)
    E, R = _tables(rng, 9, 3, 16)
    hr = _hr(rng, 9, 3, 7)
    a = ko.k_vs_all_scores("QMult", E, R, hr)
    b = ko.k_vs_all_scores_ref_form("QMult", E, R, hr)
    np.testing.assert_allclose(a, b, rtol=1e-11, atol=1e-14)
    c = ko.k_vs_all_scores("QMult", E, R, hr, normalize_relation=False)
    assert not np.allclose(a, c)


# ---------------------------------------------------------------------- Keci
class _GA:
    """Geometric algebra Cl(p,q) on bitmask blades; e_i^2=+1 for i<p, -1 for p<=i<p+q."""

    def __init__(self, p, q):
        self.p, self.q, self.n = p, q, p + q

    def blade_mul(self, a, b):
        sign = 1
        t = a >> 1
        while t:                      # count swaps to reorder
            if bin(t & b).count("1") & 1:
                sign = -sign
            t >>= 1
        common = a & b
        for i in range(self.n):
            if common >> i & 1 and i >= self.p:
                sign = -sign
        return a ^ b, sign

    def mul(self, x, y):
        out = {}
        for a, va in x.items():
            for b, vb in y.items():
                c, s = self.blade_mul(a, b)
                out[c] = out.get(c, 0.0) + s * va * vb
        return out


def _keci_bruteforce(E, R, hr, p, q, cp, cq):
    """score = <grade0,1 of (h r), t> + sum of grade-2 coefficients (with the
    reference's thresholds: pp needs p>=2, qq needs q>=2, pq needs both)."""
    N, d = E.shape
    r = d // (p + q + 1)
    ga = _GA(p, q)

    def mv(x, rho):
        m = {0: x[rho]}
        for i in range(p):
            m[1 << i] = x[r + rho * p + i] * cp[i]
        for j in range(q):
            m[1 << (p + j)] = x[r + r * p + rho * q + j] * cq[j]
        return m

    S = np.zeros((len(hr), N))
    for b, (hi, ri) in enumerate(hr):
        for rho in range(r):
            prod = ga.mul(mv(E[hi], rho), mv(R[ri], rho))
            g2 = 0.0
            for blade, v in prod.items():
                bits = [i for i in range(p + q) if blade >> i & 1]
                if len(bits) != 2:
                    continue
                in_p = [i < p for i in bits]
                if all(in_p):
                    g2 += v if p >= 2 else 0.0
                elif not any(in_p):
                    g2 += v if q >= 2 else 0.0
                else:
                    g2 += v if (p >= 2 and q >= 2) else 0.0
            for e in range(N):
                t = E[e]
                s = prod.get(0, 0.0) * t[rho]
                for i in range(p):
                    s += prod.get(1 << i, 0.0) * t[r + rho * p + i]
                for j in range(q):
                    s += prod.get(1 << (p + j), 0.0) * t[r + r * p + rho * q + j]
                S[b, e] += s + g2
    return S


@pytest.mark.parametrize("p,q", [(0, 0), (0, 1), (1, 0), (1, 1), (2, 0), (0, 2), (2, 2), (3, 2), (1, 3)])
def test_keci_vs_geometric_algebra(p, q):
    rng = np.random.default_rng(10 * p + q)
    r = 3
    d = r * (p + q + 1)
    E, R = _tables(rng, 6, 3, d, sd=1.0)
    hr = _hr(rng, 6, 3, 4)
    cp = rng.normal(size=p)
    cq = rng.normal(size=q)
    S = ko.k_vs_all_scores("Keci", E, R, hr, p=p, q=q, coeff_p=cp, coeff_q=cq)
    ref = _keci_bruteforce(E, R, hr, p, q, cp, cq)
    np.testing.assert_allclose(S, ref, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(
        ko.k_vs_all_scores_ref_form("Keci", E, R, hr, p=p, q=q, coeff_p=cp, coeff_q=cq), S, rtol=1e-10, atol=1e-12)


class _GAr(_GA):
    """Cl(p,q,r): r further bases that square to zero."""

    def __init__(self, p, q, r):
        super().__init__(p, q)
        self.r = r

    def blade_mul(self, a, b):
        if (a & b) >> (self.p + self.q):
            return a ^ b, 0
        return super().blade_mul(a, b)


def _decal_bruteforce(E, R, hr, p, q, r, cp, cq, cr):
    """score = <grade 0 and 1 of (h r), t> + the sum of the grade-2 coefficients, a bivector e_x e_y counted
    only when the family counts of x and of y are both >= 2 (the conditions of clifford.py:859-886)."""
    N, d = E.shape
    n = p + q + r
    re = d // (n + 1)
    ga = _GAr(p, q, r)
    count = [p] * p + [q] * q + [r] * r
    coeff = list(cp) + list(cq) + list(cr)

    def col(rho, i):                  # column of base i (0-based over p, then q, then r) of slot rho
        if i < p:
            return re + rho * p + i
        if i < p + q:
            return re + re * p + rho * q + (i - p)
        return re + re * p + re * q + rho * r + (i - p - q)

    def mv(x, rho):
        m = {0: x[rho]}
        for i in range(n):
            m[1 << i] = x[col(rho, i)] * coeff[i]
        return m

    S = np.zeros((len(hr), N))
    for b, (hi, ri) in enumerate(hr):
        for rho in range(re):
            prod = ga.mul(mv(E[hi], rho), mv(R[ri], rho))
            g2 = 0.0
            for blade, v in prod.items():
                bits = [i for i in range(n) if blade >> i & 1]
                if len(bits) == 2 and count[bits[0]] >= 2 and count[bits[1]] >= 2:
                    g2 += v
            for e in range(N):
                s = prod.get(0, 0.0) * E[e, rho]
                for i in range(n):
                    s += prod.get(1 << i, 0.0) * E[e, col(rho, i)]
                S[b, e] += s + g2
    return S


@pytest.mark.parametrize("p,q,r", [(0, 0, 1), (0, 0, 3), (1, 1, 1), (2, 2, 2), (3, 2, 2), (2, 0, 3), (0, 3, 2), (1, 3, 2),
                                   (2, 1, 0)])
def test_decal_vs_geometric_algebra_with_degenerate_bases(p, q, r):
    rng = np.random.default_rng(100 * p + 10 * q + r)
    re = 3
    d = re * (p + q + r + 1)
    E, R = _tables(rng, 6, 3, d, sd=1.0)
    hr = _hr(rng, 6, 3, 4)
    cp, cq, cr = rng.normal(size=p), rng.normal(size=q), rng.normal(size=r)
    kw = dict(p=p, q=q, r=r, coeff_p=cp, coeff_q=cq, coeff_r=cr)
    S = ko.k_vs_all_scores("DeCaL", E, R, hr, **kw)
    np.testing.assert_allclose(S, _decal_bruteforce(E, R, hr, p, q, r, cp, cq, cr), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(ko.k_vs_all_scores_ref_form("DeCaL", E, R, hr, **kw), S, rtol=1e-10, atol=1e-12)
    if r == 0:                        # no degenerate base: Keci
        np.testing.assert_allclose(ko.k_vs_all_scores("Keci", E, R, hr, p=p, q=q, coeff_p=cp, coeff_q=cq), S,
                                   rtol=1e-12, atol=1e-12)


def test_keci_reductions():
    rng = np.random.default_rng(5)
    E, R = _tables(rng, 8, 3, 12)
    hr = _hr(rng, 8, 3, 5)
    # (0,0) is DistMult
    np.testing.assert_allclose(ko.k_vs_all_scores("Keci", E, R, hr, p=0, q=0),
                               ko.k_vs_all_scores("DistMult", E, R, hr), rtol=1e-13)
    # (0,1) with c_q=1 is ComplEx
    np.testing.assert_allclose(ko.k_vs_all_scores("Keci", E, R, hr, p=0, q=1, coeff_q=[1.0]),
                               ko.k_vs_all_scores("ComplEx", E, R, hr), rtol=1e-12, atol=1e-15)
    # (0,1) with c_q=0 (the reference's initial value) is DistMult on the first half
    half = ko.k_vs_all_scores("DistMult", E[:, :6], R[:, :6], hr)
    np.testing.assert_allclose(ko.k_vs_all_scores("Keci", E, R, hr, p=0, q=1, coeff_q=[0.0]), half,
                               rtol=1e-13, atol=1e-16)


def test_keci_sigma_thresholds_fixture():
    """p=q=1: the e_p e_q bivector term is dropped; p=q=2: it is added."""
    with open(os.path.join(GOLD, "keci_thresholds.json")) as f:
        fx = json.load(f)
    for case in fx["cases"]:
        E = np.array(case["E"])
        R = np.array(case["R"])
        Q, bias = ko.build_query("Keci", E, R, np.array(case["hr"]), p=case["p"], q=case["q"],
                                 coeff_p=case["cp"], coeff_q=case["cq"])
        np.testing.assert_allclose(bias, case["bias"], rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(Q, case["Q"], rtol=1e-12, atol=1e-12)


# --------------------------------------------------------- torch-CPU op port
@pytest.mark.parametrize("model,d,kw", [
    ("DistMult", 8, {}), ("ComplEx", 8, {}), ("QMult", 8, {}),
    ("Keci", 12, dict(p=1, q=2, coeff_p=[0.7], coeff_q=[1.3, -0.4])),
    ("Keci", 15, dict(p=2, q=2, coeff_p=[0.7, 0.2], coeff_q=[1.3, -0.4])),
])
def test_torch_port_matches_numpy_oracle(model, d, kw):
    rng = np.random.default_rng(6)
    E, R = _tables(rng, 13, 4, d, sd=1.0)
    hr = _hr(rng, 13, 4, 6)
    want = ko.k_vs_all_scores(model, E, R, hr, **kw)
    tkw = dict(kw)
    for key in ("coeff_p", "coeff_q"):
        if key in tkw:
            tkw[key] = torch.tensor(tkw[key], dtype=torch.float64)
    got = tcp.forward_k_vs_all(model, torch.tensor(E), torch.tensor(R), torch.tensor(hr), **tkw).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


# -------------------------------------------------------------- norm layers
def test_layernorm_batchnorm_vs_torch():
    rng = np.random.default_rng(7)
    x = rng.normal(size=(5, 12))
    w, b = rng.normal(size=12), rng.normal(size=12)
    ref = torch.nn.functional.layer_norm(torch.tensor(x), (12,), torch.tensor(w), torch.tensor(b), 1e-5).numpy()
    np.testing.assert_allclose(ko.layer_norm(x, w, b), ref, rtol=1e-12, atol=1e-13)
    m, v = rng.normal(size=12), rng.uniform(0.5, 2, size=12)
    ref = torch.nn.functional.batch_norm(torch.tensor(x), torch.tensor(m), torch.tensor(v), training=False,
                                         eps=1e-5).numpy()
    np.testing.assert_allclose(ko.batch_norm_eval(x, m, v), ref, rtol=1e-12, atol=1e-13)


# ----------------------------------------------------------------- ranking
def test_rank_counts_vs_bruteforce_and_invariants():
    rng = np.random.default_rng(8)
    N = 40
    for trial in range(200):
        s = rng.integers(-3, 4, N).astype(np.float64)        # many exact ties
        t = int(rng.integers(0, N))
        filt = list(rng.integers(0, N, rng.integers(0, 12)))
        if trial % 2:
            filt.append(t)                                   # target listed in its own filter
        G, T, TL = ko.filtered_rank_counts(s, t, filt)
        assert 1 + G + TL == ko.filtered_rank_bruteforce(s, t, filt)
        # duplicates in the filter are idempotent
        assert (G, T, TL) == ko.filtered_rank_counts(s, t, filt + filt)
        # torch's unstable sort lands inside [lo, hi]
        sm = torch.tensor(s).clone()
        if filt:
            sm[torch.tensor(filt)] = -np.inf
        sm[t] = s[t]
        _, order = torch.sort(sm[None, :], dim=1, descending=True)
        pos = int(torch.where(order[0] == t)[0].item()) + 1
        assert 1 + G <= pos <= 1 + G + T
    # empty filter: plain rank
    s = np.array([0.1, 0.5, 0.3, 0.5])
    assert ko.filtered_rank_counts(s, 2, []) == (2, 0, 0)
    assert ko.filtered_rank_counts(s, 3, None) == (0, 1, 1)
    # -inf never outranks a finite target
    assert ko.filtered_rank_counts(np.array([-np.inf, 0.0, -np.inf]), 1, []) == (0, 0, 0)


def test_rank_interval_with_tolerance_against_brute_force():
    """The checker every GPU rank test leans on.  At tol = 0 it is [1 + G, 1 + G + T] of ``filtered_rank_counts``;
    at tol > 0 it is the set of ranks the target can take when every other kept score is moved anywhere within
    +-tol of its value (brute force over the two extreme placements: all down, all up)."""
    rng = np.random.default_rng(81)
    N = 30
    for trial in range(300):
        s = rng.integers(-4, 5, N).astype(np.float64) / 4.0   # multiples of 0.25: ties and near-ties
        t = int(rng.integers(0, N))
        filt = list(rng.integers(0, N, rng.integers(0, 10)))
        if trial % 3 == 0:
            filt.append(t)
        G, T, _ = ko.filtered_rank_counts(s, t, filt)
        assert ko.rank_interval_with_tolerance(s, t, filt, 0.0) == (1 + G, 1 + G + T)
        tol = float(rng.choice([0.1, 0.25, 0.3, 0.6]))
        lo, hi = ko.rank_interval_with_tolerance(s, t, filt, tol)
        keep = np.ones(N, bool)
        keep[np.asarray(filt, dtype=int)] = False
        keep[t] = False
        # best case for the target: everybody else as low as allowed, and the target wins every tie
        best = 1 + sum(1 for e in range(N) if keep[e] and s[e] - tol > s[t])
        # worst case: everybody else as high as allowed, and the target loses every tie
        worst = 1 + sum(1 for e in range(N) if keep[e] and s[e] + tol >= s[t])
        assert (lo, hi) == (best, worst)
        assert lo <= 1 + G and 1 + G + T <= hi                # the exact interval lies inside


def test_evaluator_port_matches_closed_form_without_ties():
    rng = np.random.default_rng(9)
    N, Rn, d = 50, 5, 8
    E, R = _tables(rng, N, Rn, d, sd=1.0)
    triples = np.stack([rng.integers(0, N, 64), rng.integers(0, Rn, 64), rng.integers(0, N, 64)], axis=1)
    er = {}
    for h, r, t in triples:
        er.setdefault((int(h), int(r)), []).append(int(t))
    ranks = tcp.evaluate_entity_prediction("ComplEx", torch.tensor(E), torch.tensor(R), triples, er, 16)
    S = ko.k_vs_all_scores("ComplEx", E, R, triples[:, :2])
    want = ko.filtered_ranks(S, triples[:, 2], [er[(int(h), int(r))] for h, r, _ in triples])
    assert ranks == list(want)
    m = ko.metrics_from_ranks(ranks)
    assert m["MRR"] == pytest.approx(sum(1.0 / r for r in ranks) / len(ranks))
    assert m["H@3"] == sum(r <= 3 for r in ranks) / len(ranks)


def test_relation_prediction_literal_fixture_and_torch_sequence():
    """The relation-prediction loop as the reference literally behaves (evaluator.py:440-471): the hand-computed
    fixture pins scores, masked columns, ranks and the IndexError; random inputs pin the numpy closed form against
    the reference's torch op sequence (mask with -inf, full sort, where)."""
    with open(os.path.join(GOLD, "relation_prediction_literal.json")) as f:
        fx = json.load(f)
    E, Rel = np.array(fx["E"], dtype=np.float64), np.array(fx["Rel"], dtype=np.float64)
    ee = {(int(k[0]), int(k[1])): v for k, v in fx["ee_vocab"]}
    trip = np.array(fx["triples"])
    S = ko.k_vs_all_scores("DistMult", E, Rel, trip[:, [0, 2]])
    np.testing.assert_array_equal(S, np.array(fx["scores"], dtype=np.float64))
    assert list(ko.relation_prediction_ranks("DistMult", E, Rel, trip, ee)) == fx["ranks"]
    assert list(ko.relation_prediction_ranks("DistMult", E, Rel, trip, {})) == fx["unfiltered_ranks"]
    assert tcp.evaluate_relation_prediction("DistMult", torch.tensor(E), torch.tensor(Rel), trip, ee, 3) == fx["ranks"]
    bad = np.array([fx["index_error_triple"]])
    with pytest.raises(IndexError):
        ko.relation_prediction_ranks("DistMult", E, Rel, bad, ee)
    with pytest.raises(IndexError):
        tcp.evaluate_relation_prediction("DistMult", torch.tensor(E), torch.tensor(Rel), bad, ee, 3)
    # random: tails below the number of relations, as the literal loop needs
    rng = np.random.default_rng(12)
    N, Rn, d = 60, 9, 8
    E, R = _tables(rng, N, Rn, d, sd=1.0)
    triples = np.stack([rng.integers(0, N, 80), rng.integers(0, Rn, 80), rng.integers(0, Rn, 80)], axis=1)
    ee = {}
    for h, r, t in triples:
        ee.setdefault((int(h), int(t)), []).append(int(r))
    got = tcp.evaluate_relation_prediction("ComplEx", torch.tensor(E), torch.tensor(R), triples, ee, 32)
    assert got == list(ko.relation_prediction_ranks("ComplEx", E, R, triples, ee))


# -------------------------------------------------------------- top-k, BCE
def test_topk_vs_bruteforce_and_torch():
    rng = np.random.default_rng(11)
    s = rng.normal(size=(6, 30))
    v, idx = ko.topk(s, 5)
    tv, tidx = torch.topk(torch.tensor(s), 5, dim=1)
    np.testing.assert_array_equal(idx, tidx.numpy())
    np.testing.assert_array_equal(v, tv.numpy())
    for b in range(6):
        assert list(idx[b]) == sorted(range(30), key=lambda e: (-s[b, e], e))[:5]
    np.testing.assert_allclose(ko.sigmoid(v), torch.sigmoid(tv).numpy(), rtol=1e-14)


@pytest.mark.parametrize("eps", [0.0, 0.1])
def test_bce_multihot_vs_torch_dense(eps):
    rng = np.random.default_rng(12)
    B, N = 7, 23
    s = rng.normal(0, 3, (B, N))
    pos = [list(rng.integers(0, N, rng.integers(0, 6))) for _ in range(B)]
    y = ko.dense_multihot(pos, N, eps, dtype=np.float64)
    ref = torch.nn.functional.binary_cross_entropy_with_logits(torch.tensor(s), torch.tensor(y)).item()
    assert ko.bce_multihot(s, pos, eps) == pytest.approx(ref, rel=1e-12)


# ------------------------------------------------------------ bf16 / int8
@pytest.mark.parametrize("eps", [0.0, 0.1])
def test_bce_backward_vs_torch_autograd(eps):
    rng = np.random.default_rng(13)
    B, N, d = 9, 31, 12
    Q = torch.tensor(rng.standard_normal((B, d)), requires_grad=True)
    E = torch.tensor(rng.standard_normal((N, d)), requires_grad=True)
    bias = torch.tensor(rng.standard_normal(B), requires_grad=True)
    positives = [sorted(set(rng.integers(0, N, rng.integers(0, 6)).tolist())) for _ in range(B)]
    y = torch.from_numpy(ko.dense_multihot(positives, N, eps, dtype=np.float64))
    loss = torch.nn.functional.binary_cross_entropy_with_logits(Q @ E.T + bias[:, None], y)
    (2.5 * loss).backward()
    dQ, dbias, dE = ko.bce_multihot_backward(Q.detach().numpy(), bias.detach().numpy(), E.detach().numpy(), positives,
                                             eps, grad_out=2.5)
    np.testing.assert_allclose(dQ, Q.grad.numpy(), rtol=1e-10, atol=1e-14)
    np.testing.assert_allclose(dbias, bias.grad.numpy(), rtol=1e-10, atol=1e-14)
    np.testing.assert_allclose(dE, E.grad.numpy(), rtol=1e-10, atol=1e-14)


def test_query_builder_backward_vs_torch_autograd():
    """Central differences of the oracle's query builder against autograd through a direct torch transcription
    of three interactions (elementwise product; complex product; Hamilton product after the consecutive-group
    normaliser of the relation)."""
    rng = np.random.default_rng(17)
    N, R, B, d = 11, 4, 9, 8
    E, Rel = rng.standard_normal((N, d)), rng.standard_normal((R, d))
    hr = np.stack([rng.integers(0, N, B), rng.integers(0, R, B)], axis=1)
    dQ = rng.standard_normal((B, d))

    def distmult(h, r):
        return h * r

    def complex_(h, r):
        m = d // 2
        return torch.cat([h[:, :m] * r[:, :m] - h[:, m:] * r[:, m:], h[:, :m] * r[:, m:] + h[:, m:] * r[:, :m]], dim=1)

    def qmult(h, r):
        r = torch.nn.functional.normalize(r.view(B, d // 4, 4), p=2, dim=2).view(B, d)
        a, b, c, dd = torch.hsplit(h, 4)
        p, q, u, v = torch.hsplit(r, 4)
        return torch.cat([a * p - b * q - c * u - dd * v, a * q + b * p + c * v - dd * u,
                          a * u - b * v + c * p + dd * q, a * v + b * u - c * q + dd * p], dim=1)

    for model, fn in (("DistMult", distmult), ("ComplEx", complex_), ("QMult", qmult)):
        Et, Rt = torch.tensor(E, requires_grad=True), torch.tensor(Rel, requires_grad=True)
        Q = fn(Et[torch.from_numpy(hr[:, 0])], Rt[torch.from_numpy(hr[:, 1])])
        np.testing.assert_allclose(Q.detach().numpy(), ko.build_query(model, E, Rel, hr)[0], rtol=1e-12, atol=1e-12)
        (Q * torch.from_numpy(dQ)).sum().backward()
        dE, dR, _ = ko.build_query_backward(model, E, Rel, hr, dQ)
        np.testing.assert_allclose(dE, Et.grad.numpy(), rtol=1e-7, atol=1e-8)
        np.testing.assert_allclose(dR, Rt.grad.numpy(), rtol=1e-7, atol=1e-8)


def test_query_builder_backward_through_the_normalisation_layers_vs_torch_autograd():
    """The same check with torch.nn.LayerNorm (its weight and bias included) and with BatchNorm1d(affine=False)
    in eval mode between the lookups and the interaction, as base_model.py:381-383 places them."""
    rng = np.random.default_rng(23)
    N, R, B, d = 9, 3, 7, 8
    E, Rel = rng.standard_normal((N, d)), rng.standard_normal((R, d))
    hr = np.stack([rng.integers(0, N, B), rng.integers(0, R, B)], axis=1)
    dQ = rng.standard_normal((B, d))
    m = d // 2

    def complex_(h, r):
        return torch.cat([h[:, :m] * r[:, :m] - h[:, m:] * r[:, m:], h[:, :m] * r[:, m:] + h[:, m:] * r[:, :m]], dim=1)

    ln_h, ln_r = torch.nn.LayerNorm(d).double(), torch.nn.LayerNorm(d).double()
    with torch.no_grad():
        for ln in (ln_h, ln_r):
            ln.weight.copy_(torch.from_numpy(rng.uniform(0.5, 1.5, d)))
            ln.bias.copy_(torch.from_numpy(rng.normal(0, 0.3, d)))
    bn_h, bn_r = torch.nn.BatchNorm1d(d, affine=False).double().eval(), torch.nn.BatchNorm1d(d, affine=False).double().eval()
    with torch.no_grad():
        for bn in (bn_h, bn_r):
            bn.running_mean.copy_(torch.from_numpy(rng.normal(0, 0.2, d)))
            bn.running_var.copy_(torch.from_numpy(rng.uniform(0.5, 2.0, d)))
    cases = (
        ({"kind": "LayerNorm", "eps": ln_h.eps, "h_weight": ln_h.weight.detach().numpy(),
          "h_bias": ln_h.bias.detach().numpy(), "r_weight": ln_r.weight.detach().numpy(),
          "r_bias": ln_r.bias.detach().numpy()}, ln_h, ln_r),
        ({"kind": "BatchNorm1d", "eps": bn_h.eps, "h_mean": bn_h.running_mean.numpy(), "h_var": bn_h.running_var.numpy(),
          "r_mean": bn_r.running_mean.numpy(), "r_var": bn_r.running_var.numpy()}, bn_h, bn_r))
    for norm, mod_h, mod_r in cases:
        Et, Rt = torch.tensor(E, requires_grad=True), torch.tensor(Rel, requires_grad=True)
        Q = complex_(mod_h(Et[torch.from_numpy(hr[:, 0])]), mod_r(Rt[torch.from_numpy(hr[:, 1])]))
        np.testing.assert_allclose(Q.detach().numpy(), ko.build_query("ComplEx", E, Rel, hr, norm=norm)[0],
                                   rtol=1e-12, atol=1e-12)
        (Q * torch.from_numpy(dQ)).sum().backward()
        dE, dR, extra = ko.build_query_backward("ComplEx", E, Rel, hr, dQ, norm=norm)
        np.testing.assert_allclose(dE, Et.grad.numpy(), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(dR, Rt.grad.numpy(), rtol=1e-6, atol=1e-7)
        if norm["kind"] == "LayerNorm":
            for key, prm in (("h_weight", mod_h.weight), ("h_bias", mod_h.bias), ("r_weight", mod_r.weight),
                             ("r_bias", mod_r.bias)):
                np.testing.assert_allclose(extra[key], prm.grad.numpy(), rtol=1e-6, atol=1e-7)
                prm.grad = None
        else:
            assert not any(k in extra for k in ("h_weight", "h_bias", "r_weight", "r_bias"))


def test_batchnorm_training_mode_forward_running_statistics_and_backward_vs_torch():
    """BatchNorm1d(affine=False).train(): the oracle's batch normalisation, the buffers the call leaves, and the
    gradient through the batch statistics, against torch's module and autograd in float64."""
    rng = np.random.default_rng(29)
    N, R, B, d = 7, 3, 6, 8
    E, Rel = rng.standard_normal((N, d)), rng.standard_normal((R, d))
    hr = np.stack([rng.integers(0, N, B), rng.integers(0, R, B)], axis=1)
    dQ = rng.standard_normal((B, d))
    bn_h = torch.nn.BatchNorm1d(d, affine=False).double().train()
    bn_r = torch.nn.BatchNorm1d(d, affine=False).double().train()
    with torch.no_grad():
        bn_h.running_mean.copy_(torch.from_numpy(rng.normal(0, 0.2, d)))
        bn_h.running_var.copy_(torch.from_numpy(rng.uniform(0.5, 2.0, d)))
    before = bn_h.running_mean.numpy().copy(), bn_h.running_var.numpy().copy()
    Et, Rt = torch.tensor(E, requires_grad=True), torch.tensor(Rel, requires_grad=True)
    h = bn_h(Et[torch.from_numpy(hr[:, 0])])
    r = bn_r(Rt[torch.from_numpy(hr[:, 1])])
    Q = h * r
    norm = {"kind": "BatchNorm1dTrain", "eps": bn_h.eps}
    np.testing.assert_allclose(Q.detach().numpy(), ko.build_query("DistMult", E, Rel, hr, norm=norm)[0],
                               rtol=1e-12, atol=1e-12)
    rm, rv = ko.batch_norm_running_update(E[hr[:, 0]], before[0], before[1], momentum=bn_h.momentum)
    np.testing.assert_allclose(rm, bn_h.running_mean.numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(rv, bn_h.running_var.numpy(), rtol=1e-12, atol=1e-14)
    (Q * torch.from_numpy(dQ)).sum().backward()
    dE, dR = ko.build_query_backward_batch("DistMult", E, Rel, hr, dQ, norm=norm)
    np.testing.assert_allclose(dE, Et.grad.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(dR, Rt.grad.numpy(), rtol=1e-6, atol=1e-7)


def test_dropout_masks_in_the_query_builder_vs_torch_ops():
    """Dropout with given masks on the looked-up rows (before LayerNorm) and on DistMult's h * r: forward and the
    central-difference backward against autograd through x * mask * scale written out in torch."""
    rng = np.random.default_rng(31)
    N, R, B, d = 9, 3, 7, 8
    E, Rel = rng.standard_normal((N, d)), rng.standard_normal((R, d))
    hr = np.stack([rng.integers(0, N, B), rng.integers(0, R, B)], axis=1)
    dQ = rng.standard_normal((B, d))
    keep = {k: (rng.random((B, d)) >= 0.3).astype(np.uint8) for k in ("keep_h", "keep_r", "keep_q")}
    drop = dict(keep, scale_in=1 / 0.7, scale_hidden=1 / 0.6)
    ln_h, ln_r = torch.nn.LayerNorm(d).double(), torch.nn.LayerNorm(d).double()
    norm = {"kind": "LayerNorm", "eps": ln_h.eps, "h_weight": ln_h.weight.detach().numpy(),
            "h_bias": ln_h.bias.detach().numpy(), "r_weight": ln_r.weight.detach().numpy(),
            "r_bias": ln_r.bias.detach().numpy()}
    Et, Rt = torch.tensor(E, requires_grad=True), torch.tensor(Rel, requires_grad=True)
    h = ln_h(Et[torch.from_numpy(hr[:, 0])] * torch.from_numpy(keep["keep_h"]) * (1 / 0.7))
    r = ln_r(Rt[torch.from_numpy(hr[:, 1])] * torch.from_numpy(keep["keep_r"]) * (1 / 0.7))
    Q = (h * r) * torch.from_numpy(keep["keep_q"]) * (1 / 0.6)
    np.testing.assert_allclose(Q.detach().numpy(), ko.build_query("DistMult", E, Rel, hr, norm=norm, dropout=drop)[0],
                               rtol=1e-12, atol=1e-12)
    (Q * torch.from_numpy(dQ)).sum().backward()
    dE, dR, _ = ko.build_query_backward("DistMult", E, Rel, hr, dQ, norm=norm, dropout=drop)
    np.testing.assert_allclose(dE, Et.grad.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(dR, Rt.grad.numpy(), rtol=1e-6, atol=1e-7)


def test_bf16_round_vs_torch():
    rng = np.random.default_rng(13)
    x = np.concatenate([rng.normal(0, 1, 5000), rng.normal(0, 1e-20, 100), [0.0, -0.0, 1.0, 3.3895314e38]])
    x = x.astype(np.float32)
    ref = torch.tensor(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(ko.bf16_round(x), ref)
    np.testing.assert_array_equal(ko.bf16_from_bits(ko.bf16_bits(x)), ref)


def test_int8_rows_closed_form():
    rng = np.random.default_rng(14)
    x = rng.normal(0, 0.1, (20, 16)).astype(np.float32)
    x[3] = 0.0
    q, s = ko.quantize_int8_rows(x)
    assert q.dtype == np.int8 and np.abs(q).max() <= 127
    assert np.all(np.abs(q[np.arange(20) != 3]).max(axis=1) == 127)
    assert np.all(q[3] == 0) and s[3] == 0.0
    err = np.abs(ko.dequantize_int8_rows(q, s) - x)
    assert np.all(err <= 0.5 * s[:, None] * (1 + 1e-6))


def test_vocab_csr_against_a_hand_written_fixture_and_set_identities():
    # 7 triples (h, r, t), one duplicate, one pair with three tails given out of order
    triples = [(2, 1, 5), (0, 0, 3), (2, 1, 4), (2, 1, 5), (1, 0, 3), (2, 1, 0), (0, 1, 3)]
    assert ko.vocab(triples, "er") == {(2, 1): [5, 4, 5, 0], (0, 0): [3], (1, 0): [3], (0, 1): [3]}
    assert ko.vocab(triples, "re") == {(1, 5): [2, 2], (0, 3): [0, 1], (1, 4): [2], (1, 0): [2], (1, 3): [0]}
    assert ko.vocab(triples, "ee") == {(2, 5): [1, 1], (0, 3): [0, 1], (2, 4): [1], (1, 3): [0], (2, 0): [1]}
    keys, row_ptr, col = ko.vocab_csr(triples, "er", range_b=2)          # R = 2: key = 2h + r
    assert keys.tolist() == [0, 1, 2, 5] and row_ptr.tolist() == [0, 1, 2, 3, 6] and col.tolist() == [3, 3, 3, 0, 4, 5]
    keys, row_ptr, col = ko.vocab_csr(triples, "re", range_b=6)          # N = 6: key = 6r + t
    assert keys.tolist() == [3, 6, 9, 10, 11] and row_ptr.tolist() == [0, 2, 3, 4, 5, 6]
    assert col.tolist() == [0, 1, 2, 0, 2, 2]
    # identities on random data: the rows partition the distinct triples
    rng = np.random.default_rng(3)
    t = np.stack([rng.integers(0, 9, 300), rng.integers(0, 4, 300), rng.integers(0, 9, 300)], axis=1)
    for kind, rb, (a, b, v) in (("er", 4, (0, 1, 2)), ("re", 9, (1, 2, 0)), ("ee", 9, (0, 2, 1))):
        keys, row_ptr, col = ko.vocab_csr(t, kind, rb)
        assert np.all(np.diff(keys) > 0) and row_ptr[0] == 0 and row_ptr[-1] == len(col)
        rebuilt = {(int(k) // rb, int(k) % rb, int(c)) for i, k in enumerate(keys) for c in col[row_ptr[i]:row_ptr[i + 1]]}
        assert rebuilt == {(int(x[a]), int(x[b]), int(x[v])) for x in t}
        assert len(col) == len(rebuilt)
        for i in range(len(keys)):
            assert np.all(np.diff(col[row_ptr[i]:row_ptr[i + 1]]) > 0)


_LP_CASES = [("OMult", 16, {}), ("OMult", 24, {"normalize_relation": False}), ("DistMult", 12, {}), ("ComplEx", 12, {}), ("QMult", 16, {}), ("QMult", 16, {"normalize_relation": False}),
             ("Keci", 12, {"p": 0, "q": 0}), ("Keci", 12, {"p": 0, "q": 1}), ("Keci", 12, {"p": 1, "q": 1}),
             ("Keci", 12, {"p": 2, "q": 0}), ("Keci", 12, {"p": 0, "q": 2}), ("Keci", 15, {"p": 2, "q": 2}),
             ("Keci", 18, {"p": 3, "q": 2}), ("Keci", 18, {"p": 1, "q": 4}),
             ("DeCaL", 14, {"p": 2, "q": 2, "r": 2}), ("DeCaL", 16, {"p": 3, "q": 1, "r": 3}),
             ("DeCaL", 12, {"p": 0, "q": 0, "r": 2}), ("DeCaL", 12, {"p": 1, "q": 1, "r": 1})]


@pytest.mark.parametrize("model,d,kw", _LP_CASES)
def test_triple_scores_and_head_direction_agree_with_the_kvsall_oracle(model, d, kw):
    """One triple, three routes: the per-triple formula, column t of the tail-direction scores of (h, r),
    column h of the head-direction scores of (r, t).  The tail direction is pinned above."""
    rng = np.random.default_rng(d + len(kw))
    N, R, n = 23, 5, 40
    E, Rel = rng.standard_normal((N, d)), rng.standard_normal((R, d))
    kw = dict(kw)
    if model in ("Keci", "DeCaL"):
        kw["coeff_p"] = rng.standard_normal(kw["p"]) + 1.0
        kw["coeff_q"] = rng.standard_normal(kw["q"]) + 1.0
    if model == "DeCaL":
        kw["coeff_r"] = rng.standard_normal(kw["r"]) + 1.0
    triples = np.stack([rng.integers(0, N, n), rng.integers(0, R, n), rng.integers(0, N, n)], axis=1)
    per_triple = ko.triple_scores(model, E, Rel, triples, **kw)
    tails = ko.k_vs_all_scores(model, E, Rel, triples[:, :2], **kw)
    np.testing.assert_allclose(per_triple, tails[np.arange(n), triples[:, 2]], rtol=1e-11, atol=1e-12)
    heads = ko.all_head_scores(model, E, Rel, triples[:, 1:], **kw)
    assert heads.shape == (n, N)
    np.testing.assert_allclose(heads[np.arange(n), triples[:, 0]], per_triple, rtol=1e-11, atol=1e-12)
    # every other column too: score(x, r, t) for a replaced head
    for x in (0, N - 1):
        swapped = triples.copy()
        swapped[:, 0] = x
        np.testing.assert_allclose(heads[:, x], ko.triple_scores(model, E, Rel, swapped, **kw), rtol=1e-11, atol=1e-12)


def test_complex_triple_score_is_the_hermitian_product():
    rng = np.random.default_rng(5)
    E, Rel = rng.standard_normal((9, 10)), rng.standard_normal((3, 10))
    triples = np.stack([rng.integers(0, 9, 20), rng.integers(0, 3, 20), rng.integers(0, 9, 20)], axis=1)
    z = lambda x: x[:, :5] + 1j * x[:, 5:]
    want = (z(E[triples[:, 0]]) * z(Rel[triples[:, 1]]) * np.conj(z(E[triples[:, 2]]))).sum(axis=1).real
    np.testing.assert_allclose(ko.triple_scores("ComplEx", E, Rel, triples), want, rtol=1e-12)


def test_lp_metrics_closed_form():
    m = ko.lp_metrics([1, 4, 11], [2, 1, 3])
    assert m["H@1"] == pytest.approx(2 / 6) and m["H@3"] == pytest.approx(4 / 6) and m["H@10"] == pytest.approx(5 / 6)
    assert m["MRR"] == pytest.approx((1 + 1 / 4 + 1 / 11 + 1 / 2 + 1 + 1 / 3) / 6)


def test_ensemble_scores_fixture_and_invariances():
    A = np.array([[0.0, 2.0, 4.0]])
    B = np.array([[10.0, 0.0, 5.0]])
    got = ko.ensemble_scores([A, B], weights=[0.25, 0.75])
    np.testing.assert_allclose(got, [[0.75, 0.125, 0.625]], rtol=1e-7)      # 0.25*[0,.5,1] + 0.75*[1,0,.5]
    np.testing.assert_allclose(ko.ensemble_scores([A, B], weighted_averaging=False), [[0.5, 0.25, 0.75]], rtol=1e-7)
    np.testing.assert_allclose(ko.ensemble_scores([A, B], weights=[1, 1], normalize_scores=False), A + B)
    rng = np.random.default_rng(0)
    S1, S2 = rng.standard_normal((6, 40)), rng.standard_normal((6, 40))
    base = ko.ensemble_scores([S1, S2], weights=[0.4, 0.6])
    moved = ko.ensemble_scores([3.0 * S1 - 7.0, S2], weights=[0.4, 0.6])      # min-max removes a positive affine map
    np.testing.assert_allclose(moved, base, atol=1e-7)
    assert base.min() >= 0.0 and base.max() <= 1.0 + 1e-12


def test_octonion_table_is_a_composition_algebra():
    """A wrong sign or index in the 8x8 table breaks at least one of these identities."""
    rng = np.random.default_rng(11)
    x, y = rng.standard_normal((50, 8)), rng.standard_normal((50, 8))
    mul = lambda a, b: np.concatenate(ko.octonion_product_blocks(a, b), axis=1)
    norm = lambda a: np.sqrt((a * a).sum(1))
    np.testing.assert_allclose(norm(mul(x, y)), norm(x) * norm(y), rtol=1e-12)           # |xy| = |x||y|
    conj = x * np.array([1, -1, -1, -1, -1, -1, -1, -1.0])
    xc = mul(x, conj)
    np.testing.assert_allclose(xc[:, 0], (x * x).sum(1), rtol=1e-12)                      # x conj(x) = |x|^2
    np.testing.assert_allclose(xc[:, 1:], 0.0, atol=1e-12)
    eye = np.eye(8)
    for i in range(1, 8):
        np.testing.assert_allclose(mul(eye[i:i + 1], eye[i:i + 1]), -eye[0:1], atol=0)    # e_i^2 = -1
        np.testing.assert_allclose(mul(eye[0:1], eye[i:i + 1]), eye[i:i + 1], atol=0)     # 1 is the unit
        np.testing.assert_allclose(mul(eye[i:i + 1], eye[0:1]), eye[i:i + 1], atol=0)
        for j in range(1, 8):
            if i != j:                                                                    # imaginary units anticommute
                np.testing.assert_allclose(mul(eye[i:i + 1], eye[j:j + 1]), -mul(eye[j:j + 1], eye[i:i + 1]), atol=0)
    np.testing.assert_allclose(mul(x, mul(x, y)), mul(mul(x, x), y), rtol=1e-10, atol=1e-10)   # alternativity
    np.testing.assert_allclose(mul(mul(x, y), y), mul(x, mul(y, y)), rtol=1e-10, atol=1e-10)
    # parts 0-3 form the quaternions with the Hamilton product pinned above
    q1, q2 = rng.standard_normal((20, 4)), rng.standard_normal((20, 4))
    pad = lambda q: np.concatenate([q, np.zeros_like(q)], axis=1)
    got = mul(pad(q1), pad(q2))
    np.testing.assert_allclose(got[:, :4], np.concatenate(ko.hamilton_product_blocks(q1, q2), axis=1), rtol=1e-12)
    np.testing.assert_allclose(got[:, 4:], 0.0, atol=0)
    # normaliser: unit octonions, block layout (element g of each of the 8 blocks)
    r = rng.standard_normal((5, 24))
    rn = ko.octonion_normalize(r)
    np.testing.assert_allclose(sum(p * p for p in ko.octonion_parts(rn)), 1.0, rtol=1e-12)


def test_multi_hop_scores_on_a_hand_made_score_table():
    # 3 entities, 2 relations; T[r][h] = scores of (h, r, ?) over the 3 entities
    T = {0: np.array([[0.9, 0.1, 0.5], [0.2, 0.8, 0.3], [0.4, 0.6, 0.7]]),
         1: np.array([[0.3, 0.7, 0.2], [0.6, 0.1, 0.9], [0.5, 0.5, 0.4]])}
    atom = lambda heads, r: T[r][np.asarray(heads)]
    mh = lambda *a, **kw: ko.multi_hop_scores(atom, *a, **kw)
    np.testing.assert_allclose(mh("1p", (0, (0,))), [0.9, 0.1, 0.5])
    # 2p, k=2, min: substitutions of (0, r0, ?) = entity 0 (0.9), entity 2 (0.5);
    # answers = max(min(0.9, T1[0]), min(0.5, T1[2])) = max([.3,.7,.2], [.5,.5,.4]) = [.5,.7,.4]
    np.testing.assert_allclose(mh("2p", (0, (0, 1)), tnorm="min", k=2), [0.5, 0.7, 0.4])
    # prod: max([.27,.63,.18], [.25,.25,.2]) = [.27,.63,.2]
    np.testing.assert_allclose(mh("2p", (0, (0, 1)), tnorm="prod", k=2), [0.27, 0.63, 0.2])
    np.testing.assert_allclose(mh("2i", ((0, (0,)), (1, (1,))), tnorm="min"), [0.6, 0.1, 0.5])
    np.testing.assert_allclose(mh("2in", ((0, (0,)), (1, (1, "n"))), tnorm="min"), [0.4, 0.1, 0.1])
    np.testing.assert_allclose(mh("2u", ((0, (0,)), (1, (1,)), ("u",)), tnorm="min"), [0.9, 0.1, 0.9])
    np.testing.assert_allclose(mh("2u", ((0, (0,)), (1, (1,)), ("u",)), tnorm="prod"), [0.96, 0.19, 0.95])
    # ip, k=1, min: 2i = [.6,.1,.5] -> entity 0 (0.6); min(0.6, T0[0]) = [.6,.1,.5]
    np.testing.assert_allclose(mh("ip", (((0, (0,)), (1, (1,))), (0,)), tnorm="min", k=1), [0.6, 0.1, 0.5])
    # pi, k=1, min: (0,r0) top = entity 0 (.9); 2p = min(.9, T1[0]) = [.3,.7,.2]; with (2, r0) = [.4,.6,.7] -> [.3,.6,.2]
    np.testing.assert_allclose(mh("pi", ((0, (0, 1)), (2, (0,))), tnorm="min", k=1), [0.3, 0.6, 0.2])
    # De Morgan with the standard negation: not(a or b) = not a and not b
    a, b = T[0][0], T[1][1]
    for norm in ("min", "prod"):
        np.testing.assert_allclose(ko.neg_norm(ko.t_conorm(a, b, norm), 0.0),
                                   ko.t_norm(ko.neg_norm(a, 0.0), ko.neg_norm(b, 0.0), norm), rtol=1e-12)
    np.testing.assert_allclose(ko.neg_norm(a, 0.0, "sugeno"), 1 - a)          # lambda = 0 is the standard negation
    np.testing.assert_allclose(ko.neg_norm(a, 1.0, "yager"), 1 - a)
