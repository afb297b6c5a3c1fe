"""The reference's op sequence for KvsAll scoring / filtered rank / top-k on torch CPU.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  ``bench.py`` times these
functions as its ``cpu_baseline`` (kind "port"); tests use them for the
placement an unstable ``torch.sort`` gives a tied target.

The reference evaluates on CPU (``dicee/executer.py:256-257``) by running, per
batch, 1-6 narrow ``torch.mm``/``einsum`` calls, a per-row Python loop of
``-inf`` fills, one full descending ``torch.sort`` and a per-row ``torch.where``
(``dicee/evaluation/evaluator.py:484-508``); ``predict_topk`` runs the same
scoring followed by ``torch.topk`` (``dicee/knowledge_graph_embeddings.py:397-401``).
The functions below issue the same torch calls in the same order on plain
tensors; nothing of the reference package is imported.
"""
from __future__ import annotations

import numpy as np
import torch


def _quaternion_normalizer(x):
    # dicee/models/quaternion.py:97-100
    shape = x.shape
    x = x.view(*shape[:-1], -1, 4)
    x = torch.nn.functional.normalize(x, p=2, dim=-1)
    return x.view(*shape)


def k_vs_all_score(model, emb_h, emb_r, emb_E, p=0, q=0, coeff_p=None, coeff_q=None,
                   normalize_relation=True, hidden=None):
    """[B,N] scores with the reference's per-model sequence of torch ops.  ``hidden``: what stands for
    ``hidden_dropout(hidden_normalizer(.))`` around DistMult's ``h * r`` (real.py:32); identity when None."""
    if model == "DistMult":                      # dicee/models/real.py:32
        hr_ = emb_h * emb_r
        return torch.mm(hr_ if hidden is None else hidden(hr_), emb_E.transpose(1, 0))
    if model == "ComplEx":                       # dicee/models/complex.py:254-264
        hr_, hi_ = torch.hsplit(emb_h, 2)
        rr_, ri_ = torch.hsplit(emb_r, 2)
        tr, ti = torch.hsplit(emb_E, 2)
        tr, ti = tr.transpose(1, 0), ti.transpose(1, 0)
        a = torch.mm(hr_ * rr_, tr)
        b = torch.mm(hr_ * ri_, ti)
        c = torch.mm(hi_ * rr_, ti)
        d = torch.mm(hi_ * ri_, tr)
        return a + b + c - d
    if model == "QMult":                         # dicee/models/quaternion.py:138-156
        if normalize_relation:
            emb_r = _quaternion_normalizer(emb_r)
        a_h, b_h, c_h, d_h = torch.hsplit(emb_h, 4)
        a_r, b_r, c_r, d_r = torch.hsplit(emb_r, 4)
        r_val = a_h * a_r - b_h * b_r - c_h * c_r - d_h * d_r
        i_val = a_h * b_r + b_h * a_r + c_h * d_r - d_h * c_r
        j_val = a_h * c_r - b_h * d_r + c_h * a_r + d_h * b_r
        k_val = a_h * d_r + b_h * c_r - c_h * b_r + d_h * a_r
        t0, t1, t2, t3 = (t.transpose(1, 0) for t in torch.hsplit(emb_E, 4))
        return torch.mm(r_val, t0) + torch.mm(i_val, t1) + torch.mm(j_val, t2) + torch.mm(k_val, t3)
    if model in ("Keci", "CKeci"):               # dicee/models/clifford.py:258-305
        B, d = emb_h.shape
        N = emb_E.shape[0]
        r = d // (p + q + 1)

        def split(x):
            n = x.shape[0]
            return (x[:, :r], x[:, r:r + r * p].reshape(n, r, p), x[:, r + r * p:].reshape(n, r, q))
        h0, hp, hq = split(emb_h)
        r0, rp, rq = split(emb_r)
        if p > 0:
            hp, rp = hp * coeff_p, rp * coeff_p
        if q > 0:
            hq, rq = hq * coeff_q, rq * coeff_q
        t0 = emb_E[:, :r]
        out = torch.einsum("br,er->be", h0 * r0, t0)
        if p > 0:
            tp = emb_E[:, r:r + r * p].view(N, r, p)
            out = out + torch.einsum("brp,er->be", hp * rp, t0) \
                + torch.einsum("brp,erp->be", torch.einsum("br,brp->brp", h0, rp), tp) \
                + torch.einsum("brp,erp->be", torch.einsum("brp,br->brp", hp, r0), tp)
        if q > 0:
            tq = emb_E[:, d - r * q:].view(N, r, q)
            out = out + torch.einsum("brq,erq->be", torch.einsum("br,brq->brq", h0, rq), tq) \
                + torch.einsum("brq,erq->be", torch.einsum("brq,br->brq", hq, r0), tq) \
                - torch.einsum("brq,er->be", hq * rq, t0)
        if p >= 2:
            iu = torch.triu_indices(p, p, offset=1)
            spp = torch.einsum("nrp,nrx->nrpx", hp, rp) - torch.einsum("nrx,nrp->nrpx", hp, rp)
            out = out + spp[:, :, iu[0], iu[1]].sum(dim=[1, 2]).unsqueeze(-1)
        if q >= 2:
            iu = torch.triu_indices(q, q, offset=1)
            sqq = torch.einsum("nrp,nrx->nrpx", hq, rq) - torch.einsum("nrx,nrp->nrpx", hq, rq)
            out = out + sqq[:, :, iu[0], iu[1]].sum(dim=[1, 2]).unsqueeze(-1)
        if p >= 2 and q >= 2:
            spq = torch.einsum("nrp,nrq->nrpq", hp, rq) - torch.einsum("nrq,nrp->nrpq", hq, rp)
            out = out + spq.sum(dim=[1, 2, 3]).unsqueeze(-1)
        return out
    raise ValueError(model)


def forward_k_vs_all(model, E, R, x, norm_h=None, norm_r=None, **kw):
    """``BaseKGE.forward`` for ``x`` of shape [B,2] (base_model.py:328-336, :377-384).  ``norm_h`` / ``norm_r``:
    the modules ``normalize_head_entity_embeddings`` / ``normalize_relation_embeddings`` (base_model.py:283-294),
    applied to the looked-up rows as at :381-383."""
    emb_h = torch.nn.functional.embedding(x[:, 0], E)
    emb_r = torch.nn.functional.embedding(x[:, 1], R)
    if norm_h is not None:
        emb_h = norm_h(emb_h)
    if norm_r is not None:
        emb_r = norm_r(emb_r)
    return k_vs_all_score(model, emb_h, emb_r, E, **kw)


def evaluate_entity_prediction(model, E, R, triples, er_vocab, batch_size, **kw):
    """``Evaluator._evaluate_entity_prediction`` (evaluator.py:473-510): list of ranks."""
    ranks = []
    n = len(triples)
    for i in range(0, n, batch_size):
        data_batch = triples[i:i + batch_size]
        e1_idx_r_idx = torch.LongTensor(np.ascontiguousarray(data_batch[:, [0, 1]]))
        e2_idx = torch.tensor(np.ascontiguousarray(data_batch[:, 2]))
        with torch.no_grad():
            predictions = forward_k_vs_all(model, E, R, e1_idx_r_idx, **kw)
        for j in range(data_batch.shape[0]):
            id_e, id_r, id_e_target = (int(v) for v in data_batch[j])
            filt = er_vocab.get((id_e, id_r), [])
            target_value = predictions[j, id_e_target].item()
            predictions[j, filt] = -np.inf
            predictions[j, id_e_target] = target_value
        _, sort_idxs = torch.sort(predictions, dim=1, descending=True)
        for j in range(data_batch.shape[0]):
            rank = torch.where(sort_idxs[j] == e2_idx[j])[0].item() + 1
            ranks.append(rank)
    return ranks


def evaluate_relation_prediction(model, E, R, triples, ee_vocab, batch_size, **kw):
    """``Evaluator._evaluate_relation_prediction`` (evaluator.py:440-471): list of ranks.  The (head, tail) pair
    goes through ``forward_k_vs_all`` as the reference passes it; torch raises IndexError when a tail id is not a
    valid row of the relation table."""
    ranks = []
    n = len(triples)
    for i in range(0, n, batch_size):
        data_batch = triples[i:i + batch_size]
        e1_idx_e2_idx = torch.LongTensor(np.ascontiguousarray(data_batch[:, [0, 2]]))
        r_idx = torch.LongTensor(np.ascontiguousarray(data_batch[:, 1]))
        with torch.no_grad():
            predictions = forward_k_vs_all(model, E, R, e1_idx_e2_idx, **kw)
        for j in range(data_batch.shape[0]):
            filt = ee_vocab.get((int(data_batch[j][0]), int(data_batch[j][2])), [])
            target_value = predictions[j, r_idx[j]].item()
            predictions[j, filt] = -np.inf
            predictions[j, r_idx[j]] = target_value
        _, sort_idxs = torch.sort(predictions, dim=1, descending=True)
        for j in range(data_batch.shape[0]):
            rank = torch.where(sort_idxs[j] == r_idx[j])[0].item() + 1
            ranks.append(rank)
    return ranks


def predict_topk_indices(model, E, R, hr_pairs, topk, batch_size, **kw):
    """``KGE.predict_missing_tail_entity(..., return_indices=True)``
    (knowledge_graph_embeddings.py:374-411): ([P,k] scores, [P,k] int64 ids)."""
    P = hr_pairs.shape[0]
    scores = torch.zeros(P, topk)
    indices = torch.zeros(P, topk, dtype=torch.long)
    for i in range(0, P, batch_size):
        batch_hr = hr_pairs[i:i + batch_size]
        batch_scores = forward_k_vs_all(model, E, R, batch_hr, **kw)
        s, idx = torch.topk(batch_scores, topk, dim=1)
        scores[i:i + batch_size] = s
        indices[i:i + batch_size] = idx
    return scores, indices


def kvsall_bce_step(model, E, R, x, positives, label_smoothing=0.0, **kw):
    """``training_step`` forward + loss (base_model.py:25-46,138) with the dense
    multi-hot target of ``KvsAll.__getitem__`` (dataset_classes.py:354-361)."""
    N = E.shape[0]
    ys = []
    for idx in positives:
        y = torch.zeros(N, dtype=E.dtype)
        y[torch.as_tensor(np.asarray(idx, dtype=np.int64))] = 1.0
        if label_smoothing:
            y = y * (1 - label_smoothing) + (1 / N)
        ys.append(y)
    y = torch.stack(ys)
    yhat = forward_k_vs_all(model, E, R, x, **kw)
    return torch.nn.BCEWithLogitsLoss()(yhat, y)
