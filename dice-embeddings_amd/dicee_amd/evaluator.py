"""Filtered link-prediction evaluation through the fused rank kernel.

Mirrors dicee's ``Evaluator`` for the KvsAll entity-prediction route
(dicee/evaluation/evaluator.py:114-198 routing, :363-392 ``eval_with_vs_all``, :394-438
``evaluate_lp_k_vs_all``, :473-510 the rank loop) and its metric reduction
(dicee/evaluation/utils.py:73-132).  Where the reference scores a batch, masks it row by row in
Python and sorts every row, this evaluator makes one fused kernel call per batch and receives three
counters per query.

Tie rule.  The reference's rank of a tied target is whatever position an unstable ``torch.sort``
gives it; every such position lies in ``[1 + n_greater, 1 + n_greater + n_equal]``.  ``tie`` picks
the representative reported here: ``"stable"`` (default; what a stable descending sort gives:
ties ordered by entity id), ``"optimistic"``, ``"pessimistic"`` or ``"mean"``.
"""
import json
import os
from types import SimpleNamespace

import numpy as np
import torch

from .csr import FilterCSR

ALL_HITS_RANGE = list(range(1, 11))


def create_hits_dict(hits_range=None):
    return {i: [] for i in (hits_range or ALL_HITS_RANGE)}


def update_hits(hits, rank, hits_range=None):
    for level in (hits_range or ALL_HITS_RANGE):
        if rank <= level:
            hits[level].append(1.0)


def compute_metrics_from_ranks_simple(ranks, num_triples, hits_dict):
    """dicee/evaluation/utils.py:73-98: H@k = #{rank <= k} / n, MRR = float64 mean of reciprocals."""
    hit_1 = sum(hits_dict.get(1, [])) / num_triples if 1 in hits_dict else 0.0
    hit_3 = sum(hits_dict.get(3, [])) / num_triples if 3 in hits_dict else 0.0
    hit_10 = sum(hits_dict.get(10, [])) / num_triples if 10 in hits_dict else 0.0
    mean_reciprocal_rank = np.mean(1.0 / np.array(ranks))
    return {"H@1": hit_1, "H@3": hit_3, "H@10": hit_10, "MRR": mean_reciprocal_rank}


def ranks_from_counts(n_greater, n_equal, n_equal_lower, tie="stable"):
    g = n_greater.to(torch.int64)
    if tie == "stable":
        return 1 + g + n_equal_lower.to(torch.int64)
    if tie == "optimistic":
        return 1 + g
    if tie == "pessimistic":
        return 1 + g + n_equal.to(torch.int64)
    if tie == "mean":
        return 1 + g + n_equal.to(torch.int64) // 2
    raise ValueError(tie)


class Evaluator:
    def __init__(self, args=None, is_continual_training=False, tie="stable"):
        if args is None:
            args = SimpleNamespace(batch_size=1024, eval_model="train_val_test", scoring_technique="KvsAll",
                                   full_storage_path=None)
        elif isinstance(args, dict):
            args = SimpleNamespace(**args)
        self.args = args
        self.is_continual_training = is_continual_training
        self.er_vocab = None
        self.csr = None
        self.num_entities = None
        self.num_relations = None
        self.report = {}
        self.during_training = False
        self.tie = tie
        self.last_ranks = None

    # ------------------------------------------------------------------ filter preparation
    def vocab_preparation(self, dataset, device=None):
        """Build the filter CSR from ``dataset.er_vocab`` (dict or Future of one, evaluator.py:83-96) or,
        if the dataset has none, from its train/valid/test triples (preprocess.py:51-60): on the GPU when
        ``device`` is one (kge_csr_build), else with numpy."""
        self.num_entities = dataset.num_entities
        self.num_relations = dataset.num_relations
        er = getattr(dataset, "er_vocab", None)
        if er is not None and hasattr(er, "result"):
            er = er.result()
        if er is not None:
            self.er_vocab = er
            self.csr = FilterCSR.from_er_vocab(er, self.num_relations)
        else:
            parts = [np.asarray(s) for s in (dataset.train_set, getattr(dataset, "valid_set", None),
                                             getattr(dataset, "test_set", None)) if s is not None]
            triples = np.concatenate(parts, axis=0)
            if device is not None and torch.device(device).type == "cuda":
                on_dev = torch.from_numpy(np.ascontiguousarray(triples.astype(np.int64))).to(device)
                self.csr = FilterCSR.from_triples_gpu(on_dev, self.num_entities, self.num_relations)
            else:
                self.csr = FilterCSR.from_triples(triples, self.num_relations)

    def set_filter(self, csr_or_er_vocab, num_relations=None):
        if isinstance(csr_or_er_vocab, FilterCSR):
            self.csr = csr_or_er_vocab
        else:
            self.er_vocab = csr_or_er_vocab
            self.csr = FilterCSR.from_er_vocab(csr_or_er_vocab, num_relations)
        return self

    # ------------------------------------------------------------------ evaluation
    def eval(self, dataset, trained_model, form_of_labelling, during_training=False):
        self.during_training = during_training
        if self.csr is None:
            self.vocab_preparation(dataset, device=trained_model.entity_embeddings.weight.device)
        if self.args.scoring_technique not in ["AllvsAll", "KvsAll", "1vsSample", "KvsSample", "1vsAll"]:
            raise ValueError(f"Invalid scoring technique: {self.args.scoring_technique}")
        self.eval_with_vs_all(train_set=dataset.train_set, valid_set=getattr(dataset, "valid_set", None),
                              test_set=getattr(dataset, "test_set", None), trained_model=trained_model,
                              form_of_labelling=form_of_labelling)
        path = getattr(self.args, "full_storage_path", None)
        if not self.during_training and path:
            with open(os.path.join(path, "eval_report.json"), "w") as f:
                json.dump({k: {m: float(v) for m, v in r.items()} for k, r in self.report.items()}, f, indent=4)
        return dict(self.report)

    def eval_with_vs_all(self, *, train_set, valid_set=None, test_set=None, trained_model, form_of_labelling):
        em = self.args.eval_model or ""
        if "train" in em:
            self.report["Train"] = self.evaluate_lp_k_vs_all(
                trained_model, train_set, info=f"Evaluate {trained_model.name} on Train set",
                form_of_labelling=form_of_labelling)
        if "val" in em and valid_set is not None:
            self.report["Val"] = self.evaluate_lp_k_vs_all(
                trained_model, valid_set, f"Evaluate {trained_model.name} on Validation set",
                form_of_labelling=form_of_labelling)
        if test_set is not None and "test" in em:
            self.report["Test"] = self.evaluate_lp_k_vs_all(
                trained_model, test_set, f"Evaluate {trained_model.name} on Test set",
                form_of_labelling=form_of_labelling)

    def evaluate_lp_k_vs_all(self, model, triple_idx, info=None, form_of_labelling=None):
        """Filtered link prediction with KvsAll scoring -> ``{'H@1','H@3','H@10','MRR'}``."""
        if form_of_labelling == "RelationPrediction":
            raise NotImplementedError("relation prediction is outside the accelerated path")
        model.eval()
        num_triples = len(triple_idx)
        if info and not self.during_training:
            print(info + ":", end=" ")
        ranks = self._evaluate_entity_prediction(model, triple_idx, num_triples)
        assert len(triple_idx) == len(ranks) == num_triples
        hits = create_hits_dict()
        for level in ALL_HITS_RANGE:
            hits[level] = [1.0] * int(np.count_nonzero(ranks <= level))
        results = compute_metrics_from_ranks_simple(ranks, num_triples, hits)
        self.last_ranks = ranks
        if info and not self.during_training:
            print(info)
            print(results)
        return results

    def _evaluate_entity_prediction(self, model, triple_idx, num_triples):
        """Ranks (numpy int64 [n]) of the true tails; one fused kernel call per batch of
        ``args.batch_size`` triples (the batching of evaluator.py:484-486)."""
        triple_idx = np.asarray(triple_idx)
        if triple_idx.ndim != 2 or triple_idx.shape[1] != 3:
            raise ValueError("triple_idx must have shape [n, 3]")
        N, R = model.num_entities, model.num_relations
        if num_triples:
            if triple_idx[:, [0, 2]].min() < 0 or triple_idx[:, [0, 2]].max() >= N or \
                    triple_idx[:, 1].min() < 0 or triple_idx[:, 1].max() >= R:
                raise IndexError("triple_idx holds an entity or relation id outside the model's tables")
        dev = model.entity_embeddings.weight.device
        csr = self.csr
        if csr is not None and (csr.device is None or csr.device != dev):
            csr.to(dev)
        all_trip = torch.from_numpy(np.ascontiguousarray(triple_idx.astype(np.int64))).to(dev)
        out = torch.empty((num_triples,), dtype=torch.int64, device=dev)
        bs = int(self.args.batch_size)
        with torch.no_grad():
            for i in range(0, num_triples, bs):
                batch = all_trip[i:i + bs]
                x = batch[:, :2].contiguous()
                t = batch[:, 2].contiguous()
                c = model.rank_filtered(x, t, csr)
                out[i:i + bs] = ranks_from_counts(c["n_greater"], c["n_equal"], c["n_equal_lower"], self.tie)
        return out.cpu().numpy()
