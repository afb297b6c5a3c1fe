"""Filtered link-prediction evaluation through the fused rank kernel.

Mirrors dicee's ``Evaluator`` for index-encoded (non byte-pair) models
(dicee/evaluation/evaluator.py:114-198 routing, :246-272 ``eval_rank_of_head_and_tail_entity``, :363-392
``eval_with_vs_all``, :394-438 ``evaluate_lp_k_vs_all``, :440-471 the relation-prediction loop, :473-510 the
entity-prediction loop, :622-643 ``evaluate_lp``) and its metric reduction
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


_STREAM_POOLS = {}   # (device index, streams) -> the side streams of evaluations on that device


class _BatchStreams:
    """Consecutive batches of an evaluation on alternating streams.  A batch is a short chain of dependent launches
    (plan, thresholds, main loop, correction); two chains side by side fill the gaps each leaves (ComplEx, 14,541
    entities, batches of 1024: 0.117 -> 0.075 ms per batch).  What a group of batches shares (query vectors, filter
    rows, whatever the model derives lazily, such as its quantised table) is made on the caller's stream before
    ``fork()``; the first batch of a group runs on the caller's stream too; ``join()`` makes the caller's stream
    wait for all of them and makes it current again.  ``scores_per_batch`` (batch size x entities),
    when given and below a million, keeps everything on the caller's stream: a batch that small is shorter than
    what crossing streams costs (135 entities, batches of 512: 0.056 -> 0.065 ms per batch on two streams)."""

    SMALL_BATCH = 1_000_000

    def __init__(self, device, n, scores_per_batch=None):
        self.n = max(1, int(n))
        if scores_per_batch is not None and scores_per_batch < self.SMALL_BATCH:
            self.n = 1
        # (a model on the CPU has no stream: the first rank call raises what the ops raise for CPU tensors)
        self.cur = torch.cuda.current_stream(device) if torch.device(device).type == "cuda" else None
        self.device = device
        self.pool = None
        self.i = 0

    def fork(self):
        """What the caller's stream has been given so far (a group's query vectors) is visible to the side streams."""
        self.i = 0
        if self.cur is None or self.n == 1:
            return
        if self.pool is None:
            # the same few streams for every evaluation on a device: torch's allocator keeps a pool of freed blocks
            # per stream, and a fresh set of streams per evaluation would leave one behind each time
            key = (torch.device(self.device).index, self.n)
            if key not in _STREAM_POOLS:
                _STREAM_POOLS[key] = [torch.cuda.Stream(device=self.device) for _ in range(self.n)]
            self.pool = _STREAM_POOLS[key]
        for s in self.pool:
            s.wait_stream(self.cur)

    def switch(self):
        """Make the next batch's stream the current one (``join()`` gives the caller's back)."""
        self.i += 1
        if self.cur is None or self.n == 1 or self.pool is None:
            return
        if self.i == 1:
            return                      # the first batch of a group: the caller's stream, which is current
        torch.cuda.set_stream(self.pool[self.i % self.n])

    def join(self):
        if self.cur is None or self.pool is None:
            return
        torch.cuda.set_stream(self.cur)
        for s in self.pool:
            self.cur.wait_stream(s)


def rank_in_batches(model, x_all, target_all, csr, batch_size, tie="stable", streams=2, heads=False,
                    call_queries=8192):
    """Ranks (int64 tensor [n] on the model's device) of ``target_all`` [n] for the queries ``x_all`` [n,2]: one fused
    rank call per batch of ``batch_size`` queries, or per run of whole batches that together hold at least
    ``call_queries`` queries (the reference's batch size bounds the B x N score matrix it materialises,
    evaluator.py:484-508; the fused call forms no such matrix, a query's counters do not depend on what else is in
    its call, and a call's fixed cost (the plan of its correction, launches, the last round of workgroups) is paid
    once per call: ``call_queries=0`` keeps one call per batch).  What does not depend on the batching is done for many batches at a
    time: the query vectors and the filter rows of a group of batches (at most 64 batches or 256 MB of vectors; every
    row is a function of its own (h, r) pair alone, so the numbers are those of batch-wise calls) and the thresholds
    (the raw scores of the targets) come from one launch each, and a batch is then nothing but the plan of its filter
    correction, the main loop and the correction, writing its counters straight into the evaluation's arrays.  Consecutive batches run on alternating streams; the ranks are formed once at the end."""
    from . import ops
    n = int(x_all.shape[0])
    dev = x_all.device
    x_all = x_all.contiguous()
    target_all = target_all.to(dtype=torch.int64).contiguous()
    counts = {k: torch.empty((n,), dtype=dt, device=dev) for k, dt in ops._RANK_OUT}
    bs = max(1, int(batch_size))
    if call_queries and bs < int(call_queries):
        bs *= -(-int(call_queries) // bs)
    d = int(model.entity_embeddings.weight.shape[1])
    group = bs * max(1, min(64, (1 << 28) // (bs * d * 4)))
    lanes = _BatchStreams(dev, streams, min(bs, n) * model.num_entities)
    try:
        with torch.no_grad():
            for g0 in range(0, n, group):
                xs = x_all[g0:g0 + group]
                Q, bias = model.query(xs, heads=heads)
                E, scale = model.table()
                rows = csr.rows_for(xs.to(device=E.device)) if csr is not None else None
                g1 = g0 + int(xs.shape[0])
                # the thresholds of the whole group (and its counters' initial values) come from one launch as well;
                # a batch is then the plan of its filter correction, the main loop and the correction.  Query vectors
                # and filter rows come from the same (h, r) pairs, so queries that share a row share a vector.
                thr = ops.rank_thresholds(Q, bias, E, scale, target_all[g0:g1], {k: v[g0:g1] for k, v in counts.items()})
                lanes.fork()
                for i in range(0, int(xs.shape[0]), bs):
                    lanes.switch()
                    Qi = Q[i:i + bs]
                    if Qi.data_ptr() % 16:      # (bs * d not a multiple of 4: the library wants 16-byte aligned rows)
                        Qi = Qi.clone()
                    ops.rank_filtered(Qi, None, E, scale,
                                      target_all[g0 + i:g0 + i + bs], None if rows is None else rows[i:i + bs],
                                      None if csr is None else csr.row_ptr, None if csr is None else csr.col,
                                      out={k: v[g0 + i:g0 + i + bs] for k, v in counts.items()},
                                      thr=thr[i:i + bs], one_vector_per_row=True)
                lanes.join()    # before the group's vectors are released to the allocator of the caller's stream
    finally:
        lanes.join()
    return ranks_from_counts(counts["n_greater"], counts["n_equal"], counts["n_equal_lower"], tie)


class Evaluator:
    def __init__(self, args=None, is_continual_training=False, tie="stable", streams=2):
        if args is None:
            args = SimpleNamespace(batch_size=1024, eval_model="train_val_test", scoring_technique="KvsAll",
                                   full_storage_path=None)
        elif isinstance(args, dict):
            args = SimpleNamespace(**args)
        self.args = args
        self.is_continual_training = is_continual_training
        self.er_vocab = None
        self.re_vocab = None
        self.ee_vocab = None
        self.csr = None          # (head, relation) -> tails: the entity-prediction filter
        self.re_csr = None       # (relation, tail) -> heads: head direction of evaluate_lp
        self.ee_csr = None       # (head, tail) -> relations: relation prediction
        self._triples = None     # all splits, kept to build the other two vocabularies on demand
        self.num_entities = None
        self.num_relations = None
        self.report = {}
        self.during_training = False
        self.tie = tie
        self.streams = streams   # batches of an evaluation alternate over this many streams (1: the caller's only)
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
            self._triples = triples
            if device is not None and torch.device(device).type == "cuda":
                on_dev = torch.from_numpy(np.ascontiguousarray(triples.astype(np.int64))).to(device)
                self.csr = FilterCSR.from_triples_gpu(on_dev, self.num_entities, self.num_relations)
            else:
                self.csr = FilterCSR.from_triples(triples, self.num_relations)

        # the other two vocabularies, when the dataset carries them (evaluator.py:83-96)
        for attr, mine, mult in (("re_vocab", "re_csr", self.num_entities), ("ee_vocab", "ee_csr", self.num_entities)):
            v = getattr(dataset, attr, None)
            if v is not None and hasattr(v, "result"):
                v = v.result()
            if v is not None:
                setattr(self, attr, v)
                setattr(self, mine, FilterCSR.from_er_vocab(v, mult))

    def set_filter(self, csr_or_vocab, num_relations=None, kind="er"):
        """Install a filter: a ``FilterCSR`` or the reference's dict.  ``kind``: ``"er"`` (h, r) -> tails,
        ``"re"`` (r, t) -> heads, ``"ee"`` (h, t) -> relations; ``num_relations`` is the multiplier of the
        row key ``first * multiplier + second`` (the number of relations for ``"er"``, of entities otherwise)."""
        attr = {"er": "csr", "re": "re_csr", "ee": "ee_csr"}[kind]
        if isinstance(csr_or_vocab, FilterCSR):
            setattr(self, attr, csr_or_vocab)
        else:
            setattr(self, {"er": "er_vocab", "re": "re_vocab", "ee": "ee_vocab"}[kind], csr_or_vocab)
            setattr(self, attr, FilterCSR.from_er_vocab(csr_or_vocab, num_relations))
        return self

    def _other_vocab(self, kind, model):
        """``re_csr`` / ``ee_csr``, built from the dataset's triples on first use when no vocabulary was given."""
        attr = {"re": "re_csr", "ee": "ee_csr"}[kind]
        csr = getattr(self, attr)
        if csr is None:
            if self._triples is None:
                raise AssertionError(f"self.{kind}_vocab cannot be None")
            dev = model.entity_embeddings.weight.device
            N, R = model.num_entities, model.num_relations
            if dev.type == "cuda":
                on_dev = torch.from_numpy(np.ascontiguousarray(self._triples.astype(np.int64))).to(dev)
                csr = FilterCSR.from_triples_gpu(on_dev, N, R, kind=kind)
            else:
                cols = {"re": [1, 2, 0], "ee": [0, 2, 1]}[kind]
                csr = FilterCSR.from_triples(np.asarray(self._triples)[:, cols], N)
            setattr(self, attr, csr)
        return csr

    # ------------------------------------------------------------------ evaluation
    def eval(self, dataset, trained_model, form_of_labelling, during_training=False):
        """Routing of Evaluator.eval (evaluator.py:114-198) for index-encoded models: ``NegSample`` ranks heads and
        tails (``evaluate_lp``), the ``*vsAll`` / ``*vsSample`` techniques rank tails (or relations) with KvsAll
        scoring.  Byte-pair-encoded models are outside the accelerated path."""
        self.during_training = during_training
        if self.args.eval_model is None:
            return None
        if getattr(self.args, "byte_pair_encoding", False):
            raise NotImplementedError("byte-pair-encoded models are outside the accelerated path")
        if isinstance(self.args.eval_model, bool):
            print("Wrong input:RESET")
            self.args.eval_model = "train_val_test"
        if "constraint" in self.args.eval_model:
            # the reference's branch (evaluator.py:498-499) indexes range_constraints_per_rel, which is never set
            raise NotImplementedError("'constraint' in eval_model: range constraints are not part of this path")
        if self.csr is None:
            self.vocab_preparation(dataset, device=trained_model.entity_embeddings.weight.device)
        if getattr(self.args, "num_folds_for_cv", 0) and self.args.num_folds_for_cv > 1:
            return None
        splits = dict(train_set=dataset.train_set, valid_set=getattr(dataset, "valid_set", None),
                      test_set=getattr(dataset, "test_set", None), trained_model=trained_model)
        if self.args.scoring_technique == "NegSample":
            self.eval_rank_of_head_and_tail_entity(**splits)
        elif self.args.scoring_technique in ["AllvsAll", "KvsAll", "1vsSample", "KvsSample", "1vsAll"]:
            self.eval_with_vs_all(form_of_labelling=form_of_labelling, **splits)
        else:
            raise ValueError(f"Invalid scoring technique: {self.args.scoring_technique}")
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

    def eval_rank_of_head_and_tail_entity(self, *, train_set, valid_set=None, test_set=None, trained_model):
        """Evaluation of models trained with negative sampling (evaluator.py:246-272): heads and tails."""
        em = self.args.eval_model or ""
        if "train" in em:
            self.report["Train"] = self.evaluate_lp(trained_model, train_set,
                                                    f"Evaluate {trained_model.name} on Train set")
        if "val" in em and valid_set is not None:
            self.report["Val"] = self.evaluate_lp(trained_model, valid_set,
                                                  f"Evaluate {trained_model.name} of Validation set")
        if test_set is not None and "test" in em:
            self.report["Test"] = self.evaluate_lp(trained_model, test_set,
                                                   f"Evaluate {trained_model.name} of Test set")

    def evaluate_lp(self, model, triple_idx, info):
        """evaluator.py:622-643: both directions through ``link_prediction.evaluate_lp``."""
        from .link_prediction import evaluate_lp
        assert self.csr is not None, "self.er_vocab cannot be None"
        return evaluate_lp(model, triple_idx, num_entities=self.num_entities, er_vocab=self.csr,
                           re_vocab=self._other_vocab("re", model), info=None if self.during_training else info,
                           tie=self.tie, streams=self.streams)

    def evaluate_lp_k_vs_all(self, model, triple_idx, info=None, form_of_labelling=None):
        """Filtered link prediction with KvsAll scoring -> ``{'H@1','H@3','H@10','MRR'}``."""
        model.eval()
        num_triples = len(triple_idx)
        if info and not self.during_training:
            print(info + ":", end=" ")
        if form_of_labelling == "RelationPrediction":
            ranks = self._evaluate_relation_prediction(model, triple_idx, num_triples)
        else:
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

    def _evaluate_relation_prediction(self, model, triple_idx, num_triples):
        """Ranks (numpy int64 [n]) as the reference's relation-prediction loop produces them
        (evaluator.py:440-471), literally: ``forward_k_vs_all`` receives the (head, TAIL) pairs, so the tail id
        is looked up in the relation table (an ``IndexError`` when it is not below the number of relations, as
        the embedding lookup raises there), the resulting scores of all ENTITIES are masked at the columns
        listed in ``ee_vocab[(head, tail)]`` (relation ids used as column numbers) and the rank is that of
        column ``relation`` among all entity columns."""
        triple_idx = np.asarray(triple_idx)
        if triple_idx.ndim != 2 or triple_idx.shape[1] != 3:
            raise ValueError("triple_idx must have shape [n, 3]")
        N, R = model.num_entities, model.num_relations
        if num_triples:
            if triple_idx[:, 0].min() < 0 or triple_idx[:, 0].max() >= N:
                raise IndexError("index out of range in self")          # entity_embeddings(head)
            if triple_idx[:, 2].min() < 0 or triple_idx[:, 2].max() >= R:
                raise IndexError("index out of range in self")          # relation_embeddings(tail)
            if triple_idx[:, 1].min() < 0 or triple_idx[:, 1].max() >= N:
                raise IndexError(f"index {int(triple_idx[:, 1].max())} is out of bounds for dimension 1 with size {N}")
        dev = model.entity_embeddings.weight.device
        csr = self._other_vocab("ee", model)
        if csr.device is None or csr.device != dev:
            csr.to(dev)
        all_trip = torch.from_numpy(np.ascontiguousarray(triple_idx.astype(np.int64))).to(dev)
        out = rank_in_batches(model, all_trip[:, [0, 2]], all_trip[:, 1], csr, self.args.batch_size, self.tie,
                              self.streams)
        return out.cpu().numpy()

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
        out = rank_in_batches(model, all_trip[:, :2], all_trip[:, 2], csr, self.args.batch_size, self.tie,
                              self.streams)
        return out.cpu().numpy()
