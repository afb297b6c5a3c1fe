"""Filtered link prediction in both directions through the fused rank kernel.

Mirrors ``evaluate_lp`` (dicee/evaluation/link_prediction.py:351-473), the evaluation dicee runs for
models trained with negative sampling: for every test triple the true tail is ranked among
``score(h, r, x)`` and the true head among ``score(x, r, t)`` over all entities x, known answers
filtered out (``er_vocab`` for tails, ``re_vocab`` for heads), and the hit rates and the MRR are
averaged over both directions.  The reference scores ``chunk_size`` entities at a time with
``batch * chunk`` per-triple forward passes and sorts every row; here each direction of a batch is
one query build plus one fused rank call (the head direction is the same table contraction as the
tail direction, with the query vector ``Q'(r, t)``).
"""
import numpy as np
import torch

from .csr import FilterCSR
from .evaluator import rank_in_batches


def _as_csr(vocab, key_mult, device):
    if vocab is None or isinstance(vocab, FilterCSR):
        csr = vocab
    else:
        csr = FilterCSR.from_er_vocab(vocab, key_mult)           # dict (a, b) -> list of values
    if csr is not None:
        csr.to(device)
    return csr


@torch.no_grad()
def evaluate_lp(model, triple_idx, num_entities=None, er_vocab=None, re_vocab=None, info="Eval Starts",
                batch_size=128, chunk_size=1000, tie="stable", return_ranks=False, streams=2):
    """``{'H@1', 'H@3', 'H@10', 'MRR'}`` over head and tail prediction.

    ``er_vocab`` / ``re_vocab``: the reference's dicts ``(h, r) -> [t]`` / ``(r, t) -> [h]``, or ``FilterCSR``
    objects (``FilterCSR.from_triples_gpu(..., kind="er" | "re")``).  ``chunk_size`` is accepted for
    signature compatibility; nothing is chunked.  ``return_ranks``: also return (head_ranks, tail_ranks).
    ``streams``: the rank calls (two per batch, independent of one another) alternate over this many streams,
    joined before the ranks are read; 1 keeps all of them on the caller's stream."""
    assert model is not None, "Model must be provided"
    assert triple_idx is not None, "triple_idx must be provided"
    assert er_vocab is not None, "er_vocab must be provided"
    assert re_vocab is not None, "re_vocab must be provided"
    model.eval()
    from .models import IdentityClass
    if not isinstance(getattr(model, "normalize_tail_entity_embeddings", IdentityClass()), IdentityClass):
        # the reference scores every candidate through forward_triples here, i.e. against NORMALISED tail rows
        # (base_model.py:374); ranking against the table as it is would silently give other ranks
        raise NotImplementedError("evaluate_lp: models that normalise the tail row (normalization with NegSample / "
                                  "KvsSample) are not part of this path; forward_triples scores them")
    N, R = model.num_entities, model.num_relations
    assert num_entities is None or num_entities == N, "num_entities does not match the model"
    triple_idx = np.asarray(triple_idx)
    if triple_idx.ndim != 2 or triple_idx.shape[1] != 3:
        raise ValueError("triple_idx must have shape [n, 3]")
    n = len(triple_idx)
    if n and (triple_idx[:, [0, 2]].min() < 0 or triple_idx[:, [0, 2]].max() >= N or triple_idx[:, 1].min() < 0
              or triple_idx[:, 1].max() >= R):
        raise IndexError("triple_idx holds an entity or relation id outside the model's tables")
    if info:
        print(info)
        print(f"Num of triples {n}")
    dev = model.entity_embeddings.weight.device
    er = _as_csr(er_vocab, R, dev)
    re = _as_csr(re_vocab, N, dev)
    trip = torch.from_numpy(np.ascontiguousarray(triple_idx.astype(np.int64))).to(dev)
    tail_ranks = rank_in_batches(model, trip[:, :2], trip[:, 2], er, batch_size, tie, streams)
    head_ranks = rank_in_batches(model, trip[:, 1:], trip[:, 0], re, batch_size, tie, streams, heads=True)
    hr_, tr_ = head_ranks.cpu().numpy(), tail_ranks.cpu().numpy()
    divisor = float(2 * n) if n else 1.0
    results = {f"H@{k}": float((np.count_nonzero(hr_ <= k) + np.count_nonzero(tr_ <= k)) / divisor) for k in (1, 3, 10)}
    results["MRR"] = float((1.0 / hr_ + 1.0 / tr_).sum() / divisor)
    if info:
        print(results)
    return (results, (hr_, tr_)) if return_ranks else results


def _ids_of_string_triples(model, triples):
    e2i, r2i = model.entity_to_idx, model.relation_to_idx
    return np.array([[e2i[s_], r2i[p_], e2i[o_]] for s_, p_, o_ in triples], dtype=np.int64).reshape(-1, 3)


def _csr_of_string_vocab(vocab, first, second, values, key_mult, device):
    """``vocab``: dict (str, str) -> list of str, as dicee stores vocabularies of string triples; ``first`` /
    ``second`` / ``values`` are the str -> id maps of the key's two parts and of the list entries."""
    ids = {(first[a], second[b]): [values[v] for v in vs] for (a, b), vs in vocab.items()}
    return FilterCSR.from_er_vocab(ids, key_mult).to(device)


@torch.no_grad()
def evaluate_link_prediction_performance_with_reciprocals(model, triples, er_vocab, tie="stable", streams=2):
    """Tail-only filtered evaluation of string triples for models trained with reciprocal relations
    (dicee/evaluation/link_prediction.py:116-174).  ``model``: a ``KGE`` (``.model``, ``.entity_to_idx``,
    ``.relation_to_idx``); ``er_vocab``: (head str, relation str) -> list of tail strs.  Batches of
    ``model.model.args["batch_size"]`` triples, one fused rank call each."""
    from .evaluator import compute_metrics_from_ranks_simple, create_hits_dict, ALL_HITS_RANGE
    net = model.model
    net.eval()
    dev = net.entity_embeddings.weight.device
    ids = _ids_of_string_triples(model, triples)
    csr = _csr_of_string_vocab(er_vocab, model.entity_to_idx, model.relation_to_idx, model.entity_to_idx,
                               net.num_relations, dev)
    trip = torch.from_numpy(ids).to(dev)
    n = len(ids)
    bs = int(net.args.get("batch_size", 1024) or 1024)
    out = rank_in_batches(net, trip[:, :2], trip[:, 2], csr, bs, tie, streams)
    ranks = out.cpu().numpy()
    assert len(triples) == len(ranks) == n
    hits = create_hits_dict()
    for level in ALL_HITS_RANGE:
        hits[level] = [1.0] * int(np.count_nonzero(ranks <= level))
    return compute_metrics_from_ranks_simple(ranks, n, hits)


@torch.no_grad()
def evaluate_link_prediction_performance(model, triples, er_vocab, re_vocab, tie="stable", streams=2):
    """Head and tail filtered evaluation of string triples (dicee/evaluation/link_prediction.py:22-113):
    ``er_vocab`` (head str, relation str) -> tails, ``re_vocab`` (relation str, tail str) -> heads."""
    net = model.model
    dev = net.entity_embeddings.weight.device
    ids = _ids_of_string_triples(model, triples)
    er = _csr_of_string_vocab(er_vocab, model.entity_to_idx, model.relation_to_idx, model.entity_to_idx,
                              net.num_relations, dev)
    re = _csr_of_string_vocab(re_vocab, model.relation_to_idx, model.entity_to_idx, model.entity_to_idx,
                              net.num_entities, dev)
    return evaluate_lp(net, ids, net.num_entities, er, re, info=None, batch_size=int(net.args.get("batch_size", 1024) or 1024),
                       tie=tie, streams=streams)
