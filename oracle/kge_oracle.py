"""numpy oracle for dicee's KvsAll scoring and link-prediction path.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``): never imported by the
shipped package.

Every function restates, in plain numpy, what the cited reference lines compute.
Arithmetic runs in float64 unless ``dtype`` says otherwise, so the oracle is a
tighter reference than the fp32 torch code it mirrors.

Pinning status (independent checks live in ``tests/test_oracle_pins.py``)
------------------------------------------------------------------------
* ``distmult_*``      brute-force triple loop; closed form ``(h*r).e``.
* ``complex_*``       ``Re<h, r, conj(t)>`` in numpy complex128; per-triple
                      formula of ``dicee/models/complex.py:229-238``.
* ``quaternion_normalize`` unit norm of every group of 4 consecutive elements,
                      zero-vector ``eps`` case, hand-computed d=8 fixture.
* ``qmult_*``         Hamilton product against an independently built 4x4x4
                      structure-constant table and against
                      ``scipy.spatial.transform.Rotation`` composition; the
                      block-split vs consecutive-group quirk has a d=8 fixture.
* ``octonion_*`` / ``omult_query``  composition-algebra identities the sign table must satisfy:
                      |xy| = |x||y|, x conj(x) = |x|^2, e_i^2 = -1, alternativity x(xy) = (xx)y and
                      (xy)y = x(yy), the quaternion subalgebra on parts 0-3 equals the (pinned)
                      Hamilton product; per-triple score against the KvsAll column.
* ``keci_*``          (p,q)=(0,0) == DistMult; (0,1), c=1 == ComplEx; (0,1),
                      c=0 == DistMult on the first half; general (p,q) against a
                      brute-force geometric-algebra product on bitmask blades;
                      thresholds p>=2 / q>=2 / (p>=2 and q>=2) by fixtures.
* ``relation_prediction_ranks``  hand-computed fixture ``tests/golden/relation_prediction_literal.json``
                      (scores, masked columns, ranks and the IndexError case worked out on paper), and the
                      torch op sequence of ``oracle/torch_cpu_path.py`` on random inputs.
* ``decal_*``         general (p,q,r) against the same brute-force geometric-algebra product with r
                      bases that square to zero (bivector families counted under the reference's
                      ">= 2 of each" conditions); r = 0 == Keci; single-GEMM form == einsum form;
                      the head-direction vector against per-triple scores with replaced heads.
                      ``triple_scores`` for DeCaL is defined as the KvsAll column (the reference's
                      ``forward_triples`` skips the coefficients and contracts over the batch).
* ``layer_norm`` / ``batch_norm_eval``  torch.nn.functional library routines.
* ``filtered_rank_counts``  explicit masking + stable argsort brute force;
                      invariants (duplicates idempotent, -inf never outranks,
                      target never masked, empty filter); torch.sort placement
                      lies inside ``[lo, hi]``.
* ``topk``            ``numpy.argsort`` brute force; sigmoid identity.
* ``bce_multihot``    ``torch.nn.functional.binary_cross_entropy_with_logits``
                      on a dense target, with and without label smoothing.
* ``bce_multihot_backward``  torch autograd (float64) through ``binary_cross_entropy_with_logits`` of
                      ``Q @ E.T + bias`` on the dense target, with and without label smoothing.
* ``build_query_backward``  central differences of the (pinned) ``build_query`` itself, so no Jacobian is
                      derived by hand; checked against torch autograd through a torch transcription of the
                      DistMult / ComplEx / QMult (normalised) forward.
* ``bf16_round`` / ``quantize_int8_rows``  torch's bf16 cast; closed forms.
* ``triple_scores``  equal to column t of the (pinned) KvsAll scores of (h, r) for all four models
                      and every (p, q); ComplEx against complex128 ``Re<h, r, conj t>``.
* ``head_query`` / ``all_head_scores``  column h of the head-direction scores of (r, t) equals
                      ``triple_scores`` and the tail-direction score of the same triple;
                      linearity in the head row.
* ``ensemble_scores``  rows lie in [0, sum of weights]; invariance under a positive affine map of one
                      model's scores; hand-computed 2-model fixture.
* ``multi_hop_scores`` / ``t_norm`` / ``t_conorm`` / ``neg_norm``  hand-computed answers on a 3-entity score
                      table for 2p, 2i, 2in, 2u, ip, pi (min and prod norms); fuzzy-logic identities
                      (De Morgan for the standard negation, 1p of a 2p with k = N and one-hot scores).
* ``vocab`` / ``vocab_csr``  hand-written 7-triple fixture; set identities
                      (every triple recoverable from exactly one row, rows
                      partition the distinct triples).
No function is "parity unpinned" with respect to the arithmetic.  What stays
unpinned is the position an *unstable* ``torch.sort`` gives a tied target
(``dicee/evaluation/evaluator.py:503``): that is torch's behaviour, not the
reference's, and the oracle reports the admissible interval instead.
"""
from __future__ import annotations

import numpy as np

MODELS = ("DistMult", "ComplEx", "QMult", "Keci", "OMult", "DeCaL")

# --------------------------------------------------------------------------
# known-answer vocabularies
# --------------------------------------------------------------------------

_VOCAB_COLUMNS = {"er": (0, 1, 2), "re": (1, 2, 0), "ee": (0, 2, 1)}


def vocab(triples, kind="er"):
    """dict pair -> list of values, insertion order, duplicates kept: ``get_er_vocab`` /
    ``get_re_vocab`` / ``get_ee_vocab`` (dicee/read_preprocess_save_load_kg/util.py:355-385)."""
    a, b, v = _VOCAB_COLUMNS[kind]
    out = {}
    for triple in triples:
        out.setdefault((int(triple[a]), int(triple[b])), []).append(int(triple[v]))
    return out


def vocab_csr(triples, kind, range_b):
    """The same vocabulary in the layout the kernels take: rows ordered by ``a * range_b + b``, values
    sorted and de-duplicated.  Returns (keys int64, row_ptr int64, col int32)."""
    voc = vocab(triples, kind)
    pairs = sorted(voc, key=lambda ab: ab[0] * range_b + ab[1])
    keys = np.array([a * range_b + b for a, b in pairs], dtype=np.int64)
    row_ptr = np.zeros(len(pairs) + 1, dtype=np.int64)
    col = []
    for i, ab in enumerate(pairs):
        vals = sorted(set(voc[ab]))
        col.extend(vals)
        row_ptr[i + 1] = len(col)
    return keys, row_ptr, np.array(col, dtype=np.int32)


# --------------------------------------------------------------------------
# storage emulation (exists only in this build; the reference is fp32-only)
# --------------------------------------------------------------------------


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 to the nearest bf16 (ties to even), returned as fp32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    nan = np.isnan(x)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32).copy()
    out[nan] = np.nan
    return out.reshape(x.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of ``bf16_round(x)``."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def quantize_int8_rows(x: np.ndarray):
    """Per-row symmetric int8: ``scale = max|row|/127``, ``q = rint(row/scale)``."""
    x = np.asarray(x, dtype=np.float32)
    amax = np.abs(x).max(axis=1)
    scale = (amax / 127.0).astype(np.float32)
    safe = np.where(scale > 0, scale, 1.0).astype(np.float32)
    q = np.rint(x / safe[:, None]).clip(-127, 127).astype(np.int8)
    return q, scale


def dequantize_int8_rows(q: np.ndarray, scale: np.ndarray) -> np.ndarray:
    return q.astype(np.float32) * scale.astype(np.float32)[:, None]


# --------------------------------------------------------------------------
# G2: gather (+ optional normalisation)   dicee/models/base_model.py:377-384
# --------------------------------------------------------------------------


def layer_norm(x, weight, bias, eps=1e-5):
    """torch.nn.LayerNorm over the last axis (base_model.py:283-288)."""
    x = np.asarray(x, dtype=np.float64)
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * np.asarray(weight, np.float64) + np.asarray(bias, np.float64)


def batch_norm_eval(x, running_mean, running_var, eps=1e-5):
    """torch.nn.BatchNorm1d(affine=False) in eval mode (base_model.py:289-294)."""
    x = np.asarray(x, dtype=np.float64)
    return (x - np.asarray(running_mean, np.float64)) / np.sqrt(np.asarray(running_var, np.float64) + eps)


def batch_norm_train(x, eps=1e-5):
    """torch.nn.BatchNorm1d(affine=False) in training mode (base_model.py:289-294 while ``self.training``): every
    feature by the mean and the BIASED variance of the batch it is given."""
    x = np.asarray(x, dtype=np.float64)
    mu = x.mean(axis=0, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=0, keepdims=True)
    return (x - mu) / np.sqrt(var + eps)


def batch_norm_running_update(x, running_mean, running_var, momentum=0.1):
    """What the same call leaves in the module's buffers: ``(1 - momentum) * running + momentum * statistic`` with the
    batch mean and the UNBIASED batch variance (torch.nn.BatchNorm1d, training mode)."""
    x = np.asarray(x, dtype=np.float64)
    n = x.shape[0]
    mu = x.mean(axis=0)
    var_unbiased = ((x - mu) ** 2).sum(axis=0) / (n - 1)
    return ((1 - momentum) * np.asarray(running_mean, np.float64) + momentum * mu,
            (1 - momentum) * np.asarray(running_var, np.float64) + momentum * var_unbiased)


def gather_hr(E, R, hr, norm=None, dtype=np.float64, dropout=None):
    """Head / relation rows for a batch of (head_id, relation_id) pairs.

    Dropout is the identity in eval mode (base_model.py:149-151).  ``norm`` is
    None (IdentityClass) or a dict: ``{"kind": "LayerNorm", "h_weight", "h_bias",
    "r_weight", "r_bias", "eps"}`` / ``{"kind": "BatchNorm1d", "h_mean", "h_var",
    "r_mean", "r_var", "eps"}`` / ``{"kind": "BatchNorm1dTrain", "eps"}`` (the statistics of this very batch).
    ``dropout`` (training mode, base_model.py:381-383: on the looked-up rows, BEFORE the normaliser): dict with
    ``keep_h`` / ``keep_r`` ([B,d] 0/1 masks, either may be missing) and ``scale_in`` = 1 / (1 - rate); torch.nn.Dropout
    multiplies the kept elements by that scale and zeroes the others.
    """
    hr = np.asarray(hr)
    h = np.take(np.asarray(E), hr[:, 0], axis=0).astype(dtype)
    r = np.take(np.asarray(R), hr[:, 1], axis=0).astype(dtype)
    if dropout is not None:
        scale = dropout.get("scale_in", 1.0)
        if dropout.get("keep_h") is not None:
            h = (h * (np.asarray(dropout["keep_h"]) != 0) * scale).astype(dtype)
        if dropout.get("keep_r") is not None:
            r = (r * (np.asarray(dropout["keep_r"]) != 0) * scale).astype(dtype)
    if norm is not None:
        eps = norm.get("eps", 1e-5)
        if norm["kind"] == "LayerNorm":
            h = layer_norm(h, norm["h_weight"], norm["h_bias"], eps).astype(dtype)
            r = layer_norm(r, norm["r_weight"], norm["r_bias"], eps).astype(dtype)
        elif norm["kind"] == "BatchNorm1d":
            h = batch_norm_eval(h, norm["h_mean"], norm["h_var"], eps).astype(dtype)
            r = batch_norm_eval(r, norm["r_mean"], norm["r_var"], eps).astype(dtype)
        elif norm["kind"] == "BatchNorm1dTrain":
            h = batch_norm_train(h, eps).astype(dtype)
            r = batch_norm_train(r, eps).astype(dtype)
        else:
            raise NotImplementedError(norm["kind"])
    return h, r


# --------------------------------------------------------------------------
# M1 DistMult   dicee/models/real.py:19-36
# --------------------------------------------------------------------------


def distmult_query(h, r):
    return h * r


def distmult_scores_ref_form(h, r, E):
    """``mm(h*r, E^T)`` (real.py:32)."""
    return (h * r) @ np.asarray(E, dtype=h.dtype).T


# --------------------------------------------------------------------------
# M2 ComplEx   dicee/models/complex.py:240-269
# --------------------------------------------------------------------------


def complex_query(h, r):
    """Single-GEMM form: Q = [hr*rr - hi*ri | hr*ri + hi*rr]."""
    d2 = h.shape[1] // 2
    hr_, hi_ = h[:, :d2], h[:, d2:]
    rr_, ri_ = r[:, :d2], r[:, d2:]
    return np.concatenate([hr_ * rr_ - hi_ * ri_, hr_ * ri_ + hi_ * rr_], axis=1)


def complex_scores_ref_form(h, r, E):
    """The four ``torch.mm`` of complex.py:260-264, in that order."""
    E = np.asarray(E, dtype=h.dtype)
    d2 = h.shape[1] // 2
    hr_, hi_ = h[:, :d2], h[:, d2:]
    rr_, ri_ = r[:, :d2], r[:, d2:]
    tr, ti = E[:, :d2].T, E[:, d2:].T
    return (hr_ * rr_) @ tr + (hr_ * ri_) @ ti + (hi_ * rr_) @ ti - (hi_ * ri_) @ tr


# --------------------------------------------------------------------------
# M3-M5 QMult   dicee/models/quaternion.py:74-100,124-171; static_funcs.py:4-18
# --------------------------------------------------------------------------


def quaternion_normalize(x, eps=1e-12):
    """``F.normalize(x.view(B, d/4, 4), p=2, dim=-1)`` (quaternion.py:97-100).

    Groups are 4 *consecutive* elements; each is divided by ``max(||g||, eps)``.
    """
    B, d = x.shape
    g = x.reshape(B, d // 4, 4)
    n = np.sqrt((g * g).sum(axis=-1, keepdims=True))
    return (g / np.maximum(n, eps)).reshape(B, d)


def hamilton_product_blocks(h, r):
    """``quaternion_mul`` on block-split parts (static_funcs.py:13-17)."""
    d4 = h.shape[1] // 4
    a, b, c, d_ = (h[:, i * d4:(i + 1) * d4] for i in range(4))
    p, q, u, v = (r[:, i * d4:(i + 1) * d4] for i in range(4))
    r_val = a * p - b * q - c * u - d_ * v
    i_val = a * q + b * p + c * v - d_ * u
    j_val = a * u - b * v + c * p + d_ * q
    k_val = a * v + b * u - c * q + d_ * p
    return r_val, i_val, j_val, k_val


def qmult_query(h, r, normalize_relation=True):
    """Single-GEMM form: Q = [r_val | i_val | j_val | k_val].

    ``normalize_relation`` is True when the model's
    ``normalize_relation_embeddings`` is the IdentityClass (quaternion.py:138-139).
    """
    if normalize_relation:
        r = quaternion_normalize(r)
    return np.concatenate(hamilton_product_blocks(h, r), axis=1)


def qmult_scores_ref_form(h, r, E, normalize_relation=True):
    """The four ``torch.mm`` of quaternion.py:152-156."""
    E = np.asarray(E, dtype=h.dtype)
    if normalize_relation:
        r = quaternion_normalize(r)
    d4 = h.shape[1] // 4
    parts = hamilton_product_blocks(h, r)
    out = 0
    for i, part in enumerate(parts):
        out = out + part @ E[:, i * d4:(i + 1) * d4].T
    return out


# --------------------------------------------------------------------------
# OMult   dicee/models/octonion.py:5-19 (octonion_mul), :57-70 (normaliser), :112-152 (k_vs_all_score)
# --------------------------------------------------------------------------
# e_j = sum_i SIGN[j][i] * x_i * y_(i xor j): the eight lines of octonion_mul, read off term by term.
OCTONION_SIGN = np.array([
    [+1, -1, -1, -1, -1, -1, -1, -1],
    [+1, +1, +1, -1, +1, -1, -1, +1],
    [+1, -1, +1, +1, +1, +1, -1, -1],
    [+1, +1, -1, +1, +1, -1, +1, -1],
    [+1, -1, -1, -1, +1, +1, +1, +1],
    [+1, +1, -1, +1, -1, +1, -1, +1],
    [+1, +1, +1, -1, -1, +1, +1, -1],
    [+1, -1, +1, +1, -1, -1, +1, +1]], dtype=np.float64)


def octonion_parts(x):
    m = x.shape[1] // 8
    return [x[:, i * m:(i + 1) * m] for i in range(8)]


def octonion_normalize(r):
    """Each octonion (element g of the 8 blocks) divided by its norm; no epsilon (octonion.py:57-70)."""
    parts = octonion_parts(r)
    den = np.sqrt(sum(p * p for p in parts))
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.concatenate([p / den for p in parts], axis=1)


def octonion_product_blocks(x, y):
    xp, yp = octonion_parts(x), octonion_parts(y)
    return [sum(OCTONION_SIGN[j][i] * xp[i] * yp[i ^ j] for i in range(8)) for j in range(8)]


def omult_query(h, r, normalize_relation=True):
    if normalize_relation:
        r = octonion_normalize(r)
    return np.concatenate(octonion_product_blocks(h, r), axis=1)


# --------------------------------------------------------------------------
# M6-M9 Keci   dicee/models/clifford.py:4-28,105-113,162-192,258-305
# --------------------------------------------------------------------------


def keci_split(x, r, p, q):
    """``construct_cl_multivector`` (clifford.py:162-192): a0 [B,r], ap [B,r,p], aq [B,r,q]."""
    B = x.shape[0]
    a0 = x[:, :r]
    ap = x[:, r:r + r * p].reshape(B, r, p)
    aq = x[:, r + r * p:r + r * p + r * q].reshape(B, r, q)
    return a0, ap, aq


def keci_query(h, r_emb, p, q, coeff_p=None, coeff_q=None):
    """Single-GEMM form of ``Keci.k_vs_all_score``: returns (Q [B,d], bias [B]).

    Q[:, :r]               = h0 r0 + sum_i hp_i rp_i - sum_j hq_j rq_j
    Q[:, r + rho*p + i]    = h0[rho] rp[rho,i] + hp[rho,i] r0[rho]
    Q[:, r+r*p + rho*q+j]  = h0[rho] rq[rho,j] + hq[rho,j] r0[rho]
    bias = sigma_pp (p>=2) + sigma_qq (q>=2) + sigma_pq (p>=2 and q>=2).
    Both h and r parts are scaled by the coefficients (clifford.py:105-113).
    """
    B, d = h.shape
    assert d % (p + q + 1) == 0
    r = d // (p + q + 1)
    h0, hp, hq = keci_split(h, r, p, q)
    r0, rp, rq = keci_split(r_emb, r, p, q)
    if p > 0:
        cp = np.asarray(coeff_p, dtype=h.dtype).reshape(1, 1, p)
        hp, rp = hp * cp, rp * cp
    if q > 0:
        cq = np.asarray(coeff_q, dtype=h.dtype).reshape(1, 1, q)
        hq, rq = hq * cq, rq * cq
    q0 = h0 * r0 + (hp * rp).sum(axis=2) - (hq * rq).sum(axis=2)
    qp = h0[:, :, None] * rp + hp * r0[:, :, None]
    qq = h0[:, :, None] * rq + hq * r0[:, :, None]
    Q = np.concatenate([q0, qp.reshape(B, r * p), qq.reshape(B, r * q)], axis=1)
    bias = np.zeros(B, dtype=h.dtype)
    if p >= 2:
        for i in range(p - 1):
            for k in range(i + 1, p):
                bias += (hp[:, :, i] * rp[:, :, k] - hp[:, :, k] * rp[:, :, i]).sum(axis=1)
    if q >= 2:
        for j in range(q - 1):
            for k in range(j + 1, q):
                bias += (hq[:, :, j] * rq[:, :, k] - hq[:, :, k] * rq[:, :, j]).sum(axis=1)
    if p >= 2 and q >= 2:
        for i in range(p):
            for j in range(q):
                bias += (hp[:, :, i] * rq[:, :, j] - hq[:, :, j] * rp[:, :, i]).sum(axis=1)
    return Q, bias


def keci_scores_ref_form(h, r_emb, E, p, q, coeff_p=None, coeff_q=None):
    """The einsum sequence of clifford.py:258-305, term by term."""
    E = np.asarray(E, dtype=h.dtype)
    B, d = h.shape
    N = E.shape[0]
    r = d // (p + q + 1)
    h0, hp, hq = keci_split(h, r, p, q)
    r0, rp, rq = keci_split(r_emb, r, p, q)
    if p > 0:
        cp = np.asarray(coeff_p, dtype=h.dtype).reshape(1, 1, p)
        hp, rp = hp * cp, rp * cp
    if q > 0:
        cq = np.asarray(coeff_q, dtype=h.dtype).reshape(1, 1, q)
        hq, rq = hq * cq, rq * cq
    t0 = E[:, :r]
    out = np.einsum("br,er->be", h0 * r0, t0)
    if p > 0:
        tp = E[:, r:r + r * p].reshape(N, r, p)
        out = out + np.einsum("brp,er->be", hp * rp, t0) \
            + np.einsum("brp,erp->be", h0[:, :, None] * rp, tp) \
            + np.einsum("brp,erp->be", hp * r0[:, :, None], tp)
    if q > 0:
        tq = E[:, d - r * q:].reshape(N, r, q)
        out = out + np.einsum("brq,erq->be", h0[:, :, None] * rq, tq) \
            + np.einsum("brq,erq->be", hq * r0[:, :, None], tq) \
            - np.einsum("brq,er->be", hq * rq, t0)
    if p >= 2:
        iu = np.triu_indices(p, k=1)
        spp = np.einsum("nrp,nrx->nrpx", hp, rp) - np.einsum("nrx,nrp->nrpx", hp, rp)
        out = out + spp[:, :, iu[0], iu[1]].sum(axis=(1, 2))[:, None]
    if q >= 2:
        iu = np.triu_indices(q, k=1)
        sqq = np.einsum("nrp,nrx->nrpx", hq, rq) - np.einsum("nrx,nrp->nrpx", hq, rq)
        out = out + sqq[:, :, iu[0], iu[1]].sum(axis=(1, 2))[:, None]
    if p >= 2 and q >= 2:
        spq = np.einsum("nrp,nrq->nrpq", hp, rq) - np.einsum("nrq,nrp->nrpq", hq, rp)
        out = out + spq.sum(axis=(1, 2, 3))[:, None]
    return out


# --------------------------------------------------------------------------
# DeCaL: Cl(p, q, r) with r degenerate bases   dicee/models/clifford.py:579-912
# --------------------------------------------------------------------------


def decal_split(x, re, p, q, r):
    """construct_cl_multivector (clifford.py:914-953): [B,d] -> x0 [B,re], xp [B,re,p], xq [B,re,q], xk [B,re,r]."""
    B = x.shape[0]
    o1, o2, o3 = re, re + re * p, re + re * p + re * q
    return (x[:, :re], x[:, o1:o2].reshape(B, re, p), x[:, o2:o3].reshape(B, re, q),
            x[:, o3:o3 + re * r].reshape(B, re, r))


def _decal_parts(h, r_emb, p, q, r, coeff_p, coeff_q, coeff_r):
    d = h.shape[1]
    assert d % (1 + p + q + r) == 0
    re = d // (1 + p + q + r)
    h0, hp, hq, hk = decal_split(h, re, p, q, r)
    r0, rp, rq, rk = decal_split(r_emb, re, p, q, r)
    # apply_coefficients (clifford.py:901-912): base parts of head and relation scaled, scalar parts not
    if p > 0:
        c = np.asarray(coeff_p, dtype=h.dtype).reshape(1, 1, p)
        hp, rp = hp * c, rp * c
    if q > 0:
        c = np.asarray(coeff_q, dtype=h.dtype).reshape(1, 1, q)
        hq, rq = hq * c, rq * c
    if r > 0:
        c = np.asarray(coeff_r, dtype=h.dtype).reshape(1, 1, r)
        hk, rk = hk * c, rk * c
    return re, (h0, hp, hq, hk), (r0, rp, rq, rk)


def _decal_sigmas(hs, rs, p, q, r):
    """The six sigma sums of clifford.py:859-886, each present only when both of its base counts are >= 2."""
    _, hp, hq, hk = hs
    _, rp, rq, rk = rs

    def same(x, y, n):        # compute_sigma_pp / qq / rr: upper triangle of x_i y_k - x_k y_i
        return sum((x[:, :, i] * y[:, :, k] - x[:, :, k] * y[:, :, i]).sum(axis=1)
                   for i in range(n - 1) for k in range(i + 1, n))

    def cross(xa, xb, ya, yb):  # compute_sigma_pq / pr / qr: xa_i yb_j - xb_j ya_i over all pairs
        return (np.einsum("nri,nrj->n", xa, yb) - np.einsum("nrj,nri->n", xb, ya))

    out = np.zeros(hp.shape[0], dtype=hp.dtype)
    if p >= 2:
        out = out + same(hp, rp, p)
    if q >= 2:
        out = out + same(hq, rq, q)
    if r >= 2:
        out = out + same(hk, rk, r)
    if p >= 2 and q >= 2:
        out = out + cross(hp, hq, rp, rq)
    if p >= 2 and r >= 2:
        out = out + cross(hp, hk, rp, rk)
    if q >= 2 and r >= 2:
        out = out + cross(hq, hk, rq, rk)
    return out


def decal_scores_ref_form(h, r_emb, E, p, q, r, coeff_p=None, coeff_q=None, coeff_r=None):
    """DeCaL.forward_k_vs_all (clifford.py:808-899), einsum by einsum."""
    E = np.asarray(E, dtype=h.dtype)
    N = E.shape[0]
    re, (h0, hp, hq, hk), (r0, rp, rq, rk) = _decal_parts(h, r_emb, p, q, r, coeff_p, coeff_q, coeff_r)
    t0 = E[:, :re]
    out = np.einsum("br,er->be", h0 * r0, t0)
    if p > 0:
        tp = E[:, re:re + re * p].reshape(N, re, p)
        out = out + np.einsum("brp,er->be", hp * rp, t0) + np.einsum("brp,erp->be", h0[:, :, None] * rp, tp) \
            + np.einsum("brp,erp->be", hp * r0[:, :, None], tp)
    if q > 0:
        o = re + re * p
        tq = E[:, o:o + re * q].reshape(N, re, q)
        out = out + np.einsum("brq,erq->be", h0[:, :, None] * rq, tq) + np.einsum("brq,erq->be", hq * r0[:, :, None], tq) \
            - np.einsum("brq,er->be", hq * rq, t0)
    if r > 0:
        tk = E[:, E.shape[1] - re * r:].reshape(N, re, r)
        out = out + np.einsum("brk,erk->be", h0[:, :, None] * rk, tk) + np.einsum("brk,erk->be", hk * r0[:, :, None], tk)
    return out + _decal_sigmas((h0, hp, hq, hk), (r0, rp, rq, rk), p, q, r)[:, None]


def decal_query(h, r_emb, p, q, r, coeff_p=None, coeff_q=None, coeff_r=None):
    """Single-GEMM form: (Q [B,d], bias [B]) with ``forward_k_vs_all == Q @ E^T + bias``."""
    B = h.shape[0]
    re, (h0, hp, hq, hk), (r0, rp, rq, rk) = _decal_parts(h, r_emb, p, q, r, coeff_p, coeff_q, coeff_r)
    q0 = h0 * r0 + (hp * rp).sum(axis=2) - (hq * rq).sum(axis=2)
    blocks = [q0]
    for hx, rx, n in ((hp, rp, p), (hq, rq, q), (hk, rk, r)):
        blocks.append((h0[:, :, None] * rx + hx * r0[:, :, None]).reshape(B, re * n))
    return np.concatenate(blocks, axis=1), _decal_sigmas((h0, hp, hq, hk), (r0, rp, rq, rk), p, q, r)


def decal_head_query(r_emb, t, p, q, r, coeff_p=None, coeff_q=None, coeff_r=None):
    """Q' with ``forward_k_vs_all((x, rel))[tail] = Q' . E[x]``: the coefficient of every head component."""
    B = t.shape[0]
    re, (t0, tp, tq, tk), (r0, rp, rq, rk) = _decal_parts(t, r_emb, p, q, r, None if not p else np.ones(p),
                                                           None if not q else np.ones(q), None if not r else np.ones(r))
    cs = [np.asarray(c if n else [], dtype=t.dtype).reshape(1, 1, n)
          for c, n in ((coeff_p, p), (coeff_q, q), (coeff_r, r))]
    rp, rq, rk = rp * cs[0], rq * cs[1], rk * cs[2]
    q0 = r0 * t0 + (rp * tp).sum(2) + (rq * tq).sum(2) + (rk * tk).sum(2)
    qp = rp * t0[:, :, None] + r0[:, :, None] * tp
    qq = -rq * t0[:, :, None] + r0[:, :, None] * tq
    qk = r0[:, :, None] * tk
    for blk, rx, n in ((qp, rp, p), (qq, rq, q), (qk, rk, r)):
        if n >= 2:                                           # d sigma_xx / d hx_i = sum_{k>i} rx_k - sum_{k<i} rx_k
            for i in range(n):
                blk[:, :, i] += rx[:, :, i + 1:].sum(2) - rx[:, :, :i].sum(2)
    sp, sq, sk = rp.sum(2)[:, :, None], rq.sum(2)[:, :, None], rk.sum(2)[:, :, None]
    if p >= 2 and q >= 2:
        qp, qq = qp + sq, qq - sp
    if p >= 2 and r >= 2:
        qp, qk = qp + sk, qk - sp
    if q >= 2 and r >= 2:
        qq, qk = qq + sk, qk - sq
    return np.concatenate([q0, (qp * cs[0]).reshape(B, re * p), (qq * cs[1]).reshape(B, re * q),
                           (qk * cs[2]).reshape(B, re * r)], axis=1)


# --------------------------------------------------------------------------
# model dispatch
# --------------------------------------------------------------------------


def build_query(model, E, R, hr, p=0, q=0, coeff_p=None, coeff_q=None,
                normalize_relation=True, norm=None, dtype=np.float64, r=0, coeff_r=None, dropout=None):
    """(Q [B,d], bias [B]) such that ``scores = Q @ E.T + bias[:, None]``.  ``dropout``: see ``gather_hr``; its
    ``keep_q`` / ``scale_hidden`` are DistMult's dropout on ``h * r`` (real.py:32)."""
    h, r_ = gather_hr(E, R, hr, norm=norm, dtype=dtype, dropout=dropout)
    if model == "DistMult":
        Q = distmult_query(h, r_)
        if dropout is not None and dropout.get("keep_q") is not None:
            Q = (Q * (np.asarray(dropout["keep_q"]) != 0) * dropout.get("scale_hidden", 1.0)).astype(dtype)
        return Q, np.zeros(len(h), dtype)
    if model == "ComplEx":
        return complex_query(h, r_), np.zeros(len(h), dtype)
    if model == "QMult":
        return qmult_query(h, r_, normalize_relation), np.zeros(len(h), dtype)
    if model == "OMult":
        return omult_query(h, r_, normalize_relation), np.zeros(len(h), dtype)
    if model in ("Keci", "CKeci"):
        return keci_query(h, r_, p, q, coeff_p, coeff_q)
    if model == "DeCaL":
        return decal_query(h, r_, p, q, r, coeff_p, coeff_q, coeff_r)
    raise ValueError(model)


def build_query_backward(model, E, R, hr, dQ, dbias=None, step=1e-6, **kw):
    """Gradients of ``sum_b dQ[b] . Q[b] + dbias[b] * bias[b]`` (``Q, bias = build_query``) with respect to the
    entity table, the relation table and the Clifford coefficients: what autograd sends back through the
    embedding lookups and the model's interaction (dicee/models/base_model.py:377-384 and the elementwise part of
    each ``forward_k_vs_all``).  Formed by central differences in float64, one coordinate of the gathered rows at
    a time: independent of any hand-derived Jacobian (exact up to rounding for the bilinear models, ~1e-9
    relative through the normalisers).  Returns (dE [N,d], dR [R,d], {"coeff_p": ..., ...}).  With a
    ``norm=`` layer (``gather_hr``) the differences pass through it as well, row by row (LayerNorm, or BatchNorm1d
    with its running statistics: base_model.py:283-294), and the dict also holds the gradients of LayerNorm's
    parameters under ``"h_weight", "h_bias", "r_weight", "r_bias"``."""
    E = np.asarray(E, dtype=np.float64)
    R = np.asarray(R, dtype=np.float64)
    hr = np.asarray(hr)
    dQ = np.asarray(dQ, dtype=np.float64)
    B, d = dQ.shape
    db = np.zeros(B) if dbias is None else np.asarray(dbias, dtype=np.float64)
    rows_h, rows_r = E[hr[:, 0]].copy(), R[hr[:, 1]].copy()
    pairs = np.stack([np.arange(B), np.arange(B)], axis=1)
    kw = {k: (np.asarray(v, dtype=np.float64) if k.startswith("coeff") and v is not None else v) for k, v in kw.items()}

    def per_pair(h_rows, r_rows, kwargs):
        Q, bias = build_query(model, h_rows, r_rows, pairs, dtype=np.float64, **kwargs)
        return (dQ * Q).sum(axis=1) + db * bias

    dE, dR = np.zeros_like(E), np.zeros_like(R)
    for k in range(d):
        for rows, out, ids, which in ((rows_h, dE, hr[:, 0], 0), (rows_r, dR, hr[:, 1], 1)):
            plus, minus = rows.copy(), rows.copy()
            plus[:, k] += step
            minus[:, k] -= step
            if which == 0:
                g = (per_pair(plus, rows_r, kw) - per_pair(minus, rows_r, kw)) / (2 * step)
            else:
                g = (per_pair(rows_h, plus, kw) - per_pair(rows_h, minus, kw)) / (2 * step)
            np.add.at(out[:, k], ids, g)
    dcoeff = {}
    for key in ("coeff_p", "coeff_q", "coeff_r"):
        c = kw.get(key)
        if c is None or len(c) == 0:
            continue
        grad = np.zeros(len(c))
        for i in range(len(c)):
            kp, km = dict(kw), dict(kw)
            kp[key], km[key] = c.copy(), c.copy()
            kp[key][i] += step
            km[key][i] -= step
            grad[i] = ((per_pair(rows_h, rows_r, kp) - per_pair(rows_h, rows_r, km)) / (2 * step)).sum()
        dcoeff[key] = grad
    norm = kw.get("norm")
    if norm is not None and norm["kind"] == "LayerNorm":
        for key in ("h_weight", "h_bias", "r_weight", "r_bias"):
            w = np.asarray(norm[key], dtype=np.float64)
            grad = np.zeros(len(w))
            for i in range(len(w)):
                np_, nm = dict(norm), dict(norm)
                np_[key], nm[key] = w.copy(), w.copy()
                np_[key][i] += step
                nm[key][i] -= step
                kp, km = dict(kw), dict(kw)
                kp["norm"], km["norm"] = np_, nm
                grad[i] = ((per_pair(rows_h, rows_r, kp) - per_pair(rows_h, rows_r, km)) / (2 * step)).sum()
            dcoeff[key] = grad
    return dE, dR, dcoeff


def build_query_backward_batch(model, E, R, hr, dQ, dbias=None, step=1e-6, **kw):
    """``build_query_backward`` for a layer that couples the rows of the batch (``norm`` of kind
    ``"BatchNorm1dTrain"``): central differences of the WHOLE batch's ``sum_b dQ[b] . Q[b] + dbias[b] * bias[b]``, one
    coordinate of one looked-up row at a time, scattered to the tables.  O(B^2 d) work: small cases only.
    Returns (dE [N,d], dR [R,d])."""
    E = np.asarray(E, dtype=np.float64)
    R = np.asarray(R, dtype=np.float64)
    hr = np.asarray(hr)
    dQ = np.asarray(dQ, dtype=np.float64)
    B, d = dQ.shape
    db = np.zeros(B) if dbias is None else np.asarray(dbias, dtype=np.float64)
    rows_h, rows_r = E[hr[:, 0]].copy(), R[hr[:, 1]].copy()
    pairs = np.stack([np.arange(B), np.arange(B)], axis=1)

    def total(h_rows, r_rows):
        Q, bias = build_query(model, h_rows, r_rows, pairs, dtype=np.float64, **kw)
        return float((dQ * Q).sum() + (db * bias).sum())

    dE, dR = np.zeros_like(E), np.zeros_like(R)
    for b in range(B):
        for k in range(d):
            for rows, out, idx, which in ((rows_h, dE, hr[b, 0], 0), (rows_r, dR, hr[b, 1], 1)):
                keep = rows[b, k]
                rows[b, k] = keep + step
                up = total(rows_h, rows_r)
                rows[b, k] = keep - step
                down = total(rows_h, rows_r)
                rows[b, k] = keep
                out[idx, k] += (up - down) / (2 * step)
    return dE, dR


def k_vs_all_scores(model, E, R, hr, **kw):
    """``forward_k_vs_all``: [B,N] scores via the single-GEMM form."""
    dtype = kw.get("dtype", np.float64)
    Q, bias = build_query(model, E, R, hr, **kw)
    return Q @ np.asarray(E, dtype=dtype).T + bias[:, None]


def k_vs_all_scores_ref_form(model, E, R, hr, p=0, q=0, coeff_p=None, coeff_q=None,
                             normalize_relation=True, norm=None, dtype=np.float64, r=0, coeff_r=None):
    """``forward_k_vs_all`` via the reference's own multi-mm / einsum decomposition."""
    h, r_ = gather_hr(E, R, hr, norm=norm, dtype=dtype)
    if model == "DistMult":
        return distmult_scores_ref_form(h, r_, E)
    if model == "ComplEx":
        return complex_scores_ref_form(h, r_, E)
    if model == "QMult":
        return qmult_scores_ref_form(h, r_, E, normalize_relation)
    if model in ("Keci", "CKeci"):
        return keci_scores_ref_form(h, r_, E, p, q, coeff_p, coeff_q)
    if model == "DeCaL":
        return decal_scores_ref_form(h, r_, E, p, q, r, coeff_p, coeff_q, coeff_r)
    raise ValueError(model)


# --------------------------------------------------------------------------
# per-triple scores and the head direction   dicee/evaluation/link_prediction.py:351-473
# --------------------------------------------------------------------------
# ``evaluate_lp`` ranks the true tail among ``score(h, r, x)`` and the true head among
# ``score(x, r, t)`` over all entities x, scored triple by triple with the model's ``score`` /
# ``forward_triples``.  ``triple_scores`` restates those per-triple formulas; ``head_query`` is the
# vector Q'(r, t) with ``score(x, r, t) = Q' . E[x]`` for every x, so the head direction is the same
# table contraction as the tail direction.  Keci with p > 0: the reference's ``forward_triples``
# (clifford.py:525-531) contracts its ``'brp, erp -> b'`` einsums over the batch index of the tails
# as well, which couples unrelated triples of a batch; the per-triple value restated here is the one
# its own KvsAll path gives, ``forward_k_vs_all((h, r))[t]``.


def triple_scores(model, E, R, triples, p=0, q=0, coeff_p=None, coeff_q=None, normalize_relation=True,
                  dtype=np.float64, r=0, coeff_r=None):
    """score(h, r, t) for every row of ``triples`` [n,3]: DistMult.score (real.py:48-49),
    ComplEx.score (complex.py:229-238), QMult.score (quaternion.py:102-122), Keci.score
    (clifford.py:448-499), each written as explicit sums over the embedding parts."""
    E = np.asarray(E, dtype=dtype)
    R = np.asarray(R, dtype=dtype)
    triples = np.asarray(triples)
    if model == "DeCaL":
        # DeCaL.forward_triples (clifford.py:595-680) skips apply_coefficients and, like Keci's, contracts some
        # einsums over the batch; the per-triple value here is the one its KvsAll path gives, one triple at a time.
        return np.array([decal_scores_ref_form(E[t[0]:t[0] + 1], R[t[1]:t[1] + 1], E[t[2]:t[2] + 1], p, q, r,
                                               coeff_p, coeff_q, coeff_r)[0, 0] for t in triples], dtype=dtype)
    h, r, t = E[triples[:, 0]], R[triples[:, 1]], E[triples[:, 2]]
    n, d = h.shape
    if model == "DistMult":
        return (h * r * t).sum(axis=1)
    if model == "ComplEx":
        m = d // 2
        hr_, hi_, rr_, ri_, tr_, ti_ = h[:, :m], h[:, m:], r[:, :m], r[:, m:], t[:, :m], t[:, m:]
        return (hr_ * rr_ * tr_).sum(1) + (hr_ * ri_ * ti_).sum(1) + (hi_ * rr_ * ti_).sum(1) - (hi_ * ri_ * tr_).sum(1)
    if model == "QMult":
        if normalize_relation:
            r = quaternion_normalize(r)
        m = d // 4
        ha, hb, hc, hd = (h[:, i * m:(i + 1) * m] for i in range(4))
        ra, rb, rc, rd = (r[:, i * m:(i + 1) * m] for i in range(4))
        ta, tb, tc, td = (t[:, i * m:(i + 1) * m] for i in range(4))
        real = ha * ra - hb * rb - hc * rc - hd * rd
        imi = ha * rb + hb * ra + hc * rd - hd * rc
        imj = ha * rc - hb * rd + hc * ra + hd * rb
        imk = ha * rd + hb * rc - hc * rb + hd * ra
        return (real * ta).sum(1) + (imi * tb).sum(1) + (imj * tc).sum(1) + (imk * td).sum(1)
    if model == "OMult":                                     # OMult.score (octonion.py:72-110)
        if normalize_relation:
            r = octonion_normalize(r)
        return sum((e * tp).sum(1) for e, tp in zip(octonion_product_blocks(h, r), octonion_parts(t)))
    if model in ("Keci", "CKeci"):
        rr = d // (p + q + 1)
        out = np.zeros(n, dtype=dtype)
        cp = np.asarray(coeff_p if p else [], dtype=dtype)
        cq = np.asarray(coeff_q if q else [], dtype=dtype)
        for b in range(n):
            h0, hp, hq = (x[0] for x in keci_split(h[b:b + 1], rr, p, q))
            r0, rp, rq = (x[0] for x in keci_split(r[b:b + 1], rr, p, q))
            t0, tp, tq = (x[0] for x in keci_split(t[b:b + 1], rr, p, q))
            hp, rp, hq, rq = hp * cp, rp * cp, hq * cq, rq * cq          # h and r parts scaled, t parts not
            s = (h0 * r0 * t0).sum()
            s += ((hp * rp).sum(1) * t0).sum() + (h0[:, None] * rp * tp).sum() + (hp * r0[:, None] * tp).sum()
            s += -((hq * rq).sum(1) * t0).sum() + (h0[:, None] * rq * tq).sum() + (hq * r0[:, None] * tq).sum()
            if p >= 2:
                s += sum((hp[:, i] * rp[:, k] - hp[:, k] * rp[:, i]).sum() for i in range(p) for k in range(i + 1, p))
            if q >= 2:
                s += sum((hq[:, j] * rq[:, k] - hq[:, k] * rq[:, j]).sum() for j in range(q) for k in range(j + 1, q))
            if p >= 2 and q >= 2:
                s += sum((hp[:, i] * rq[:, j] - hq[:, j] * rp[:, i]).sum() for i in range(p) for j in range(q))
            out[b] = s
        return out
    raise ValueError(model)


def head_query(model, E, R, rt, p=0, q=0, coeff_p=None, coeff_q=None, normalize_relation=True, dtype=np.float64,
               r=0, coeff_r=None):
    """Q' [B,d] with ``score(x, rt[b,0], rt[b,1]) = Q'[b] . E[x]`` (no bias: every term holds the head)."""
    E = np.asarray(E, dtype=dtype)
    R = np.asarray(R, dtype=dtype)
    rt = np.asarray(rt)
    if model == "DeCaL":
        return decal_head_query(R[rt[:, 0]], E[rt[:, 1]], p, q, r, coeff_p, coeff_q, coeff_r)
    r, t = R[rt[:, 0]], E[rt[:, 1]]
    B, d = r.shape
    if model == "DistMult":
        return r * t
    if model == "ComplEx":                                   # Re<h, r, conj t> = <h, conj(r) t>
        m = d // 2
        rr_, ri_, tr_, ti_ = r[:, :m], r[:, m:], t[:, :m], t[:, m:]
        return np.concatenate([rr_ * tr_ + ri_ * ti_, rr_ * ti_ - ri_ * tr_], axis=1)
    if model == "QMult":                                     # <h (x) r, t> = <h, t (x) conj r>
        if normalize_relation:
            r = quaternion_normalize(r)
        m = d // 4
        conj = np.concatenate([r[:, :m], -r[:, m:]], axis=1)
        return np.concatenate(hamilton_product_blocks(t, conj), axis=1)
    if model == "OMult":                                     # coefficient of head part i: sum_j SIGN[j][i] y_(i^j) t_j
        if normalize_relation:
            r = octonion_normalize(r)
        yp, tp = octonion_parts(r), octonion_parts(t)
        return np.concatenate([sum(OCTONION_SIGN[j][i] * yp[i ^ j] * tp[j] for j in range(8)) for i in range(8)], axis=1)
    if model in ("Keci", "CKeci"):
        rr = d // (p + q + 1)
        r0, rp, rq = keci_split(r, rr, p, q)
        t0, tp, tq = keci_split(t, rr, p, q)
        cp = np.asarray(coeff_p if p else [], dtype=dtype).reshape(1, 1, p)
        cq = np.asarray(coeff_q if q else [], dtype=dtype).reshape(1, 1, q)
        rp, rq = rp * cp, rq * cq
        q0 = r0 * t0 + (rp * tp).sum(2) + (rq * tq).sum(2)
        qp = rp * t0[:, :, None] + r0[:, :, None] * tp
        qq = -rq * t0[:, :, None] + r0[:, :, None] * tq
        if p >= 2:                                           # d sigma_pp / d hp_i = sum_{k>i} rp_k - sum_{k<i} rp_k
            for i in range(p):
                qp[:, :, i] += rp[:, :, i + 1:].sum(2) - rp[:, :, :i].sum(2)
        if q >= 2:
            for j in range(q):
                qq[:, :, j] += rq[:, :, j + 1:].sum(2) - rq[:, :, :j].sum(2)
        if p >= 2 and q >= 2:                                # sigma_pq = sum_ij hp_i rq_j - hq_j rp_i
            qp += rq.sum(2)[:, :, None]
            qq -= rp.sum(2)[:, :, None]
        qp, qq = qp * cp, qq * cq                            # the head's own parts are scaled too
        return np.concatenate([q0, qp.reshape(B, rr * p), qq.reshape(B, rr * q)], axis=1)
    raise ValueError(model)


def all_head_scores(model, E, R, rt, **kw):
    """[B,N]: score(x, r, t) for every entity x."""
    dtype = kw.get("dtype", np.float64)
    return head_query(model, E, R, rt, **kw) @ np.asarray(E, dtype=dtype).T


def ensemble_scores(score_list, weights=None, weighted_averaging=True, normalize_scores=True):
    """Combined [B,N] scores of an ensemble (dicee/evaluation/ensemble.py:88-110): per model and row min-max
    normalisation ``(s - min) / (max - min + 1e-8)``, then the weighted sum (or the plain mean)."""
    preds = []
    for S in score_list:
        S = np.asarray(S, dtype=np.float64)
        if normalize_scores:
            lo, hi = S.min(axis=1, keepdims=True), S.max(axis=1, keepdims=True)
            S = (S - lo) / (hi - lo + 1e-8)
        preds.append(S)
    stack = np.stack(preds, axis=0)
    if weighted_averaging:
        w = np.asarray(weights, dtype=np.float64).reshape(-1, 1, 1)
        return (stack * w).sum(axis=0)
    return stack.mean(axis=0)


# --------------------------------------------------------------------------
# multi-hop query answering   dicee/knowledge_graph_embeddings.py:670-1170, dicee/abstracts.py:443-472
# --------------------------------------------------------------------------


def t_norm(a, b, tnorm="min"):
    return np.minimum(a, b) if "min" in tnorm else a * b


def t_conorm(a, b, tconorm="min"):
    return np.maximum(a, b) if "min" in tconorm else (a + b) - (a * b)


def neg_norm(a, lambda_, kind="standard"):
    if "standard" in kind:
        return 1 - a
    if "sugeno" in kind:
        return (1 - a) / (1 + lambda_ * a)
    return (1 - np.power(a, lambda_)) ** (1 / lambda_)


def _top(scores, k):
    idx = np.argsort(-scores, kind="stable")[:k]
    return scores[idx], idx


def multi_hop_scores(atom, query_type, query, tnorm="prod", neg="standard", lambda_=0.0, k=10):
    """[N] scores of every entity as answer of an EPFO query.  ``atom(heads, r)`` -> [len(heads), N] scores of
    (head, r, ?) for entity ids ``heads`` and relation ``r`` (the reference calls ``predict`` with its default
    ``logits=True``, so the norms act on logits).  A projection after a sub-query keeps the k best
    substitutions of the intermediate variable and takes, per answer, the best t-norm of
    (substitution score, next atom)."""
    def hop(prev_scores, r):                       # project: top-k substitutions, then max over them
        s, idx = _top(prev_scores, k)
        return t_norm(s[:, None], atom(list(idx), r), tnorm).max(axis=0)
    one = lambda e, r: atom([e], r)[0]
    if query_type == "1p":
        e, (r1,) = query
        return one(e, r1)
    if query_type == "2p":
        e, (r1, r2) = query
        return hop(one(e, r1), r2)
    if query_type == "3p":
        e, (r1, r2, r3) = query
        return hop(hop(one(e, r1), r2), r3)
    if query_type in ("2i", "3i", "2in", "3in", "2u"):
        parts = [q for q in query if q != ("u",)]
        vals = []
        for e, rel in parts:
            v = one(e, rel[0])
            vals.append(neg_norm(v, lambda_, neg) if rel[-1] == "n" else v)
        comb = t_conorm if query_type == "2u" else t_norm
        out = vals[0]
        for v in vals[1:]:
            out = comb(out, v, tnorm)
        return out
    if query_type in ("ip", "inp", "up"):
        inner, (r,) = query
        inner_type = {"ip": "2i", "inp": "2in", "up": "2u"}[query_type]
        return hop(multi_hop_scores(atom, inner_type, inner, tnorm, neg, lambda_, k), r)
    if query_type in ("pi", "pin", "pni"):
        (e1, rels), (e3, rel3) = query
        a1 = one(e1, rels[0])
        s, idx = _top(a1, k)
        a2 = atom(list(idx), rels[1])
        if query_type == "pni":
            a2 = neg_norm(a2, lambda_, neg)
        two_p = t_norm(s[:, None], a2, tnorm).max(axis=0)
        last = one(e3, rel3[0])
        if query_type == "pin":
            last = neg_norm(last, lambda_, neg)
        return t_norm(two_p, last, tnorm)
    raise ValueError(f"Invalid query type: {query_type}")


def lp_metrics(head_ranks, tail_ranks):
    """``evaluate_lp``'s reduction (link_prediction.py:452-468): hits count both directions over 2n,
    MRR = sum(1/head_rank + 1/tail_rank) / 2n."""
    hr_, tr_ = np.asarray(head_ranks, dtype=np.int64), np.asarray(tail_ranks, dtype=np.int64)
    n2 = float(2 * len(hr_))
    out = {f"H@{k}": float(((hr_ <= k).sum() + (tr_ <= k).sum()) / n2) for k in (1, 3, 10)}
    out["MRR"] = float((1.0 / hr_ + 1.0 / tr_).sum() / n2)
    return out


# --------------------------------------------------------------------------
# R1: filtered rank   dicee/evaluation/evaluator.py:473-510
# --------------------------------------------------------------------------


def filtered_rank_counts(scores_row, target, filt):
    """Closed form of the reference's mask + sort + where for one row.

    Returns (G, T, TL): over entities not removed by the filter (the target is
    always kept, evaluator.py:494-501), ``G`` scores strictly greater than the
    target's, ``T`` other entities tying with it, ``TL`` of those with a lower
    index.  The reference's rank lies in ``[1+G, 1+G+T]``; a stable descending
    sort gives ``1+G+TL``.
    """
    s = np.asarray(scores_row)
    N = s.shape[0]
    keep = np.ones(N, dtype=bool)
    if filt is not None and len(filt):
        keep[np.asarray(filt, dtype=np.int64)] = False
    keep[target] = True
    st = s[target]
    G = int(np.count_nonzero(keep & (s > st)))
    eq = keep & (s == st)
    eq[target] = False
    T = int(np.count_nonzero(eq))
    TL = int(np.count_nonzero(eq[:target]))
    return G, T, TL


def filtered_rank_bruteforce(scores_row, target, filt):
    """The reference's literal procedure with a *stable* descending sort."""
    s = np.array(scores_row, dtype=np.float64, copy=True)
    tv = s[target]
    if filt is not None and len(filt):
        s[np.asarray(filt, dtype=np.int64)] = -np.inf
    s[target] = tv
    order = np.argsort(-s, kind="stable")
    return int(np.where(order == target)[0][0]) + 1


def filtered_ranks(scores, targets, filters, tie="stable"):
    """Ranks for a batch. ``filters[j]`` is a sequence of entity ids (or None)."""
    out = np.empty(len(targets), dtype=np.int64)
    for j, t in enumerate(targets):
        G, T, TL = filtered_rank_counts(scores[j], int(t), filters[j])
        out[j] = 1 + G + {"stable": TL, "optimistic": 0, "pessimistic": T}[tie]
    return out


def relation_prediction_ranks(model, E, R, triples, ee_vocab, tie="stable", **kw):
    """Ranks of the reference's relation-prediction loop (dicee/evaluation/evaluator.py:440-471), literally.

    The loop hands ``(head, tail)`` pairs to ``forward_k_vs_all`` (:450-454), which looks the second column up
    in the RELATION table (base_model.py:377-384): a tail id that is not below the number of relations raises
    ``IndexError`` there.  The result holds one score per ENTITY; the loop masks the columns listed in
    ``ee_vocab[(head, tail)]`` (relation ids used as column numbers, :457-460, the target column restored) and
    takes the position of column ``relation`` in a descending sort over all entity columns (:462-467).
    ``ee_vocab``: dict ``(head, tail) -> [relation ids]`` (missing key: empty list, it is a defaultdict there).
    """
    triples = np.asarray(triples, dtype=np.int64)
    N, nR = E.shape[0], R.shape[0]
    if len(triples) and (triples[:, 2].max() >= nR or triples[:, 2].min() < 0):
        raise IndexError("index out of range in self")
    if len(triples) and (triples[:, 1].max() >= N or triples[:, 1].min() < 0):
        raise IndexError("relation id used as a column of the entity scores is out of bounds")
    S = k_vs_all_scores(model, E, R, triples[:, [0, 2]], **kw)
    filters = [list(ee_vocab.get((int(h), int(t)), [])) for h, _, t in triples]
    return filtered_ranks(S, triples[:, 1], filters, tie=tie)


def rank_interval_with_tolerance(scores_row, target, filt, tol):
    """[lo, hi] of ranks admissible when scores are only known to ``+-tol``."""
    s = np.asarray(scores_row, dtype=np.float64)
    keep = np.ones(s.shape[0], dtype=bool)
    if filt is not None and len(filt):
        keep[np.asarray(filt, dtype=np.int64)] = False
    keep[target] = False
    st = s[target]
    lo = 1 + int(np.count_nonzero(keep & (s > st + tol)))
    hi = 1 + int(np.count_nonzero(keep & (s >= st - tol)))
    return lo, hi


# --------------------------------------------------------------------------
# U1: metrics   dicee/evaluation/utils.py:73-118
# --------------------------------------------------------------------------


def metrics_from_ranks(ranks):
    ranks = np.asarray(ranks)
    n = len(ranks)
    return {
        "H@1": float(np.count_nonzero(ranks <= 1)) / n,
        "H@3": float(np.count_nonzero(ranks <= 3)) / n,
        "H@10": float(np.count_nonzero(ranks <= 10)) / n,
        "MRR": np.mean(1.0 / np.array(ranks)),
    }


# --------------------------------------------------------------------------
# K1/K2: top-k   dicee/knowledge_graph_embeddings.py:397-401,568
# --------------------------------------------------------------------------


def topk(scores, k):
    """Descending top-k per row; ties broken towards the lower index."""
    s = np.asarray(scores)
    order = np.argsort(-s, axis=1, kind="stable")[:, :k]
    return np.take_along_axis(s, order, axis=1), order


def sigmoid(x):
    x = np.asarray(x, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-x))


# --------------------------------------------------------------------------
# L1: multi-hot BCE   base_model.py:138; dataset_classes.py:354-361
# --------------------------------------------------------------------------


def softplus(x):
    x = np.asarray(x, dtype=np.float64)
    return np.maximum(x, 0.0) + np.log1p(np.exp(-np.abs(x)))


def bce_multihot(scores, positives, label_smoothing=0.0):
    """``BCEWithLogitsLoss()(scores, y)`` (mean over B*N) with ``y`` the multi-hot
    of ``positives[b]`` and the KvsAll smoothing ``y*(1-eps) + 1/N`` applied only
    when ``eps`` is non-zero (dataset_classes.py:359-360)."""
    s = np.asarray(scores, dtype=np.float64)
    B, N = s.shape
    total = softplus(s).sum()
    pos_sum = 0.0
    for b in range(B):
        idx = np.unique(np.asarray(positives[b], dtype=np.int64))
        pos_sum += s[b, idx].sum()
    if label_smoothing:
        total -= (1.0 - label_smoothing) * pos_sum + s.sum() / N
    else:
        total -= pos_sum
    return total / (B * N)


def bce_multihot_backward(Q, bias, E, positives, label_smoothing=0.0, grad_out=1.0):
    """Gradients of ``bce_multihot(Q @ E.T + bias[:, None], positives)``: what autograd computes behind
    ``loss_batch.backward()`` in the KvsAll training step (dicee/models/base_model.py:25-46).
    d loss / d score = (sigmoid(s) - y') / (B N); returns (dQ [B,d], dbias [B], dE [N,d])."""
    Q = np.asarray(Q, dtype=np.float64)
    E = np.asarray(E, dtype=np.float64)
    B, N = Q.shape[0], E.shape[0]
    s = Q @ E.T + (0.0 if bias is None else np.asarray(bias, dtype=np.float64)[:, None])
    y = dense_multihot(positives, N, label_smoothing, dtype=np.float64)
    g = grad_out * (sigmoid(s) - y) / (B * N)
    return g @ E, g.sum(axis=1), g.T @ Q


def dense_multihot(positives, N, label_smoothing=0.0, dtype=np.float32):
    y = np.zeros((len(positives), N), dtype=dtype)
    for b, idx in enumerate(positives):
        y[b, np.asarray(idx, dtype=np.int64)] = 1.0
    if label_smoothing:
        y = y * (1 - label_smoothing) + 1.0 / N
    return y
