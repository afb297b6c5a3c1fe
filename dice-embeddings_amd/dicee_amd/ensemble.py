"""Filtered link prediction of an ensemble of models without any [B, N] score matrix.

Mirrors ``evaluate_ensemble_link_prediction_performance`` (dicee/evaluation/ensemble.py:20-135): the
scores of every model are min-max normalised per query, averaged with weights (or plainly), the known
answers are filtered and the true tail is ranked.  The reference materialises and normalises one
[batch, N] matrix per model.  Here the normalisation is folded into the query vectors: with
``a_m[b] = w_m / (max_m[b] - min_m[b] + 1e-8)`` the combined score of entity e is
``sum_m a_m[b] * (Q_m[b] . E_m[e]) + const[b]``, i.e. ONE contraction of the concatenated, row-scaled
queries against the column-wise concatenation of the entity tables.  Per batch: M query builds, M fused
row min/max passes (``kge_row_minmax``), one fused filtered rank (``kge_rank_filtered``).
"""
import numpy as np
import torch

from . import ops
from .csr import FilterCSR
from .evaluator import (ALL_HITS_RANGE, compute_metrics_from_ranks_simple, create_hits_dict, ranks_from_counts)


@torch.no_grad()
def evaluate_ensemble_link_prediction_performance(models, triples, er_vocab, weights=None, batch_size=512,
                                                  weighted_averaging=True, normalize_scores=True, tie="stable",
                                                  return_ranks=False):
    """``{'H@1', 'H@3', 'H@10', 'MRR'}`` of the ensemble.  ``models``: ``dicee_amd`` models over the same entity
    and relation vocabularies, all on one GPU; ``triples`` [n,3] ids; ``er_vocab`` dict ``(h, r) -> [t]`` or a
    ``FilterCSR``."""
    n_models = len(models)
    assert n_models >= 1, "At least one model is needed."
    if weighted_averaging:
        assert weights is not None, "Weights must be provided for weighted averaging."
        assert len(weights) == n_models, "Number of weights must match number of models."
        w = [float(x) for x in weights]
    else:
        w = [1.0 / n_models] * n_models
    N, R = models[0].num_entities, models[0].num_relations
    for m in models:
        m.eval()
        assert m.num_entities == N and m.num_relations == R, "ensemble members must share their vocabularies"
    dev = models[0].entity_embeddings.weight.device
    # one fp32 table [N, sum of dims]: the dequantised tables of the members side by side
    parts = []
    for m in models:
        E, scale = m.table()
        E = E.float()
        parts.append(E if scale is None else E * scale[:, None])
    E_cat = torch.cat(parts, dim=1).contiguous() if n_models > 1 else parts[0].contiguous()
    csr = er_vocab if isinstance(er_vocab, FilterCSR) or er_vocab is None else FilterCSR.from_er_vocab(er_vocab, R)
    if csr is not None:
        csr.to(dev)
    triples = np.asarray(triples)
    num_triples = len(triples)
    trip = torch.from_numpy(np.ascontiguousarray(triples.astype(np.int64)).reshape(-1, 3)).to(dev)
    out = torch.empty((num_triples,), dtype=torch.int64, device=dev)
    for i in range(0, num_triples, int(batch_size)):
        b = trip[i:i + int(batch_size)]
        x, t = b[:, :2].contiguous(), b[:, 2].contiguous()
        qs, const = [], torch.zeros((x.shape[0],), dtype=torch.float32, device=dev)
        for m, wm in zip(models, w):
            Q, bias = m.query(x)
            if normalize_scores:
                E, scale = m.table()
                lo, hi = ops.row_minmax(Q, bias, E, scale)
                a = wm / (hi - lo + 1e-8)
                const += a * (bias - lo)
            else:
                a = torch.full_like(bias, wm)
                const += a * bias
            qs.append(Q * a[:, None])
        Q_cat = torch.cat(qs, dim=1).contiguous() if n_models > 1 else qs[0].contiguous()
        rows = csr.rows_for(x) if csr is not None else None
        c = ops.rank_filtered(Q_cat, const, E_cat, None, t, rows, csr.row_ptr if csr is not None else None,
                              csr.col if csr is not None else None)
        out[i:i + int(batch_size)] = ranks_from_counts(c["n_greater"], c["n_equal"], c["n_equal_lower"], tie)
    ranks = out.cpu().numpy()
    assert len(triples) == len(ranks) == num_triples
    hits = create_hits_dict()
    for level in ALL_HITS_RANGE:
        hits[level] = [1.0] * int(np.count_nonzero(ranks <= level))
    results = compute_metrics_from_ranks_simple(ranks, num_triples, hits)
    return (results, ranks) if return_ranks else results
