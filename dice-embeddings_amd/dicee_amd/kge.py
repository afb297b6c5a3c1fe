"""Interactive tail and head prediction on top of the fused top-k kernel.

Mirrors dicee's ``KGE`` (dicee/knowledge_graph_embeddings.py): ``predict_missing_tail_entity``
(:314-413), ``predict_missing_head_entity`` (:134-228), ``predict`` (:415-466) and ``predict_topk``
(:468-579), ``triple_score`` (:581-650) and ``answer_multi_hop_query`` (:670-1170).  The reference
scores every (x, r, t) triple through ``forward_triples`` for a missing head; here that is one
head-direction query and the same table contraction as for tails; a missing relation is scored as
the reference does it, all ``(h, x, t)`` triples through ``forward_triples`` (``kge_triple_scores``).
"""
from typing import List, Union

import torch


def _call_size(batch_size, fused_topk):
    """Queries per library call.  The reference's batch size bounds the B x N score matrix of a batch
    (knowledge_graph_embeddings.py:397-401); the fused top-k forms none and a query's top-k does not depend on what else
    is in its call, so whole batches are merged into calls of at least 4096 queries (one launch chain and one copy to
    the host per call instead of per batch; the reference's default batch is 2 pairs)."""
    batch_size = max(1, int(batch_size))
    if fused_topk and batch_size < 4096:
        batch_size *= -(-4096 // batch_size)
    return batch_size


class KGE:
    def __init__(self, path=None, model=None, entity_to_idx=None, relation_to_idx=None, model_name=None,
                 device="cuda"):
        """Either ``path``: a dicee experiment folder (``model.pt``, ``configuration.json``, ``report.json``,
        ``entity_to_idx.csv``, ``relation_to_idx.csv``; BaseInteractiveKGE.__init__, dicee/abstracts.py:170-213),
        or an in-memory ``model`` of ``dicee_amd.models`` with its two ``str -> id`` vocabularies."""
        if path is not None:
            from .loader import load_model, load_json
            self.path = path
            self.model, (entity_to_idx, relation_to_idx) = load_model(
                path, model_name=model_name or "model.pt", device=device)
            self.configs = load_json(path + "/configuration.json")
            self.configs.update(load_json(path + "/report.json"))
        else:
            if model is None or entity_to_idx is None or relation_to_idx is None:
                raise ValueError("KGE needs either `path` or `model` with both vocabularies")
            self.path = None
            self.model = model
            self.configs = dict(getattr(model, "args", {}))
        self.model.eval()
        self.entity_to_idx = dict(entity_to_idx)
        self.relation_to_idx = dict(relation_to_idx)
        self.idx_to_entity = {v: k for k, v in self.entity_to_idx.items()}
        self.idx_to_relations = {v: k for k, v in self.relation_to_idx.items()}
        self.num_entities = len(self.entity_to_idx)
        self.num_relations = len(self.relation_to_idx)
        base = [rel for rel in self.relation_to_idx if not str(rel).endswith("_inverse")]
        self.all_have_inverse = all(f"{rel}_inverse" in self.relation_to_idx for rel in base)

    # ------------------------------------------------------------------ helpers
    def _hr_pairs(self, head_entity, relation):
        if isinstance(head_entity, list):
            head = torch.LongTensor([self.entity_to_idx[i] for i in head_entity])
        else:
            head = torch.LongTensor([self.entity_to_idx[head_entity]])
        if isinstance(relation, list):
            rel = torch.LongTensor([self.relation_to_idx[i] for i in relation])
        else:
            rel = torch.LongTensor([self.relation_to_idx[relation]])
        return torch.cartesian_prod(head, rel).view(-1, 2)          # heads-major, as the reference

    def predict_missing_tail_entity(self, head_entity: Union[List[str], str], relation: Union[List[str], str],
                                    within: List[str] = None, batch_size=2, topk=1, return_indices=False):
        if within is not None:
            raise NotImplementedError("`within` needs the byte-pair-encoded path, which is outside this build")
        hr_pairs = self._hr_pairs(head_entity, relation)
        P = hr_pairs.size(0)
        T = self.num_entities
        dev = self.model.entity_embeddings.weight.device
        if return_indices:
            scores = torch.zeros(P, topk)
            indices = torch.zeros(P, topk, dtype=torch.long)
        else:
            scores = torch.zeros(P * T)
        batch_size = _call_size(batch_size, return_indices)
        for i in range(0, P, batch_size):
            batch_hr = hr_pairs[i:i + batch_size].to(dev)
            B = batch_hr.size(0)
            if return_indices:
                s, idx = self.model.topk(batch_hr, topk)          # fused: no [B,N] matrix
                scores[i:i + batch_size, :] = s.cpu()
                indices[i:i + batch_size, :] = idx.cpu()
            else:
                batch_scores = self.model(batch_hr).view(B, T)
                scores[i * T:i * T + B * T] = batch_scores.flatten().cpu()
        if return_indices:
            return scores.flatten(), indices.flatten()
        return scores

    def predict_missing_head_entity(self, relation: Union[List[str], str], tail_entity: Union[List[str], str],
                                    within: List[str] = None, batch_size=2, topk=1, return_indices=False):
        """Scores (or the top-k) of every entity as head of (?, r, t); pairs are ordered tails-major
        (``cartesian_prod(tail, relation)``).  With reciprocal relations in the vocabulary the question is asked
        as the tail of (t, r_inverse, ?), as the reference does (:166-171)."""
        if self.all_have_inverse:
            relation = [f"{relation}_inverse"] if isinstance(relation, str) else [f"{rel}_inverse" for rel in relation]
            return self.predict_missing_tail_entity(tail_entity, relation, within, batch_size, topk, return_indices)
        if within is not None:
            raise NotImplementedError("`within` needs the byte-pair-encoded path, which is outside this build")
        rel = torch.LongTensor([self.relation_to_idx[i] for i in (relation if isinstance(relation, list) else [relation])])
        tail = torch.LongTensor([self.entity_to_idx[i] for i in
                                 (tail_entity if isinstance(tail_entity, list) else [tail_entity])])
        tr_pairs = torch.cartesian_prod(tail, rel).view(-1, 2)
        P, H = tr_pairs.size(0), self.num_entities
        dev = self.model.entity_embeddings.weight.device
        if return_indices:
            scores = torch.zeros(P, topk)
            indices = torch.zeros(P, topk, dtype=torch.long)
        else:
            scores = torch.zeros(P * H)
        batch_size = _call_size(batch_size, return_indices)
        for i in range(0, P, batch_size):
            batch = tr_pairs[i:i + batch_size]
            rt = torch.stack([batch[:, 1], batch[:, 0]], dim=1).to(dev)      # the kernels take (relation, tail)
            B = rt.size(0)
            if return_indices:
                s, idx = self.model.topk(rt, topk, heads=True)
                scores[i:i + batch_size, :] = s.cpu()
                indices[i:i + batch_size, :] = idx.cpu()
            else:
                scores[i * H:i * H + B * H] = self.model.forward_all_heads(rt).flatten().cpu()
        if return_indices:
            return scores.flatten(), indices.flatten()
        return scores

    def predict_missing_relations(self, head_entity: Union[List[str], str], tail_entity: Union[List[str], str],
                                  within=None, batch_size=2, topk=1, return_indices=False):
        """Scores (or the top-k) of every relation x for (h, x, t); pairs ordered heads-major
        (``cartesian_prod(head, tail)``), every (h, x, t) triple scored by ``forward_triples`` (:229-312)."""
        if within is not None:
            raise NotImplementedError("`within` needs the byte-pair-encoded path, which is outside this build")
        head = torch.LongTensor([self.entity_to_idx[i] for i in
                                 (head_entity if isinstance(head_entity, list) else [head_entity])])
        tail = torch.LongTensor([self.entity_to_idx[i] for i in
                                 (tail_entity if isinstance(tail_entity, list) else [tail_entity])])
        ht_pairs = torch.cartesian_prod(head, tail).view(-1, 2)
        P, R = ht_pairs.size(0), self.num_relations
        dev = self.model.entity_embeddings.weight.device
        relation = torch.arange(0, R)
        if return_indices:
            scores = torch.zeros(P, topk)
            indices = torch.zeros(P, topk, dtype=torch.long)
        else:
            scores = torch.zeros(P * R)
        for i in range(0, P, batch_size):
            batch = ht_pairs[i:i + batch_size]
            B = batch.size(0)
            triples = torch.stack([batch[:, 0].repeat_interleave(R), relation.repeat(B),
                                   batch[:, 1].repeat_interleave(R)], dim=1).to(dev)
            with torch.no_grad():
                batch_scores = self.model.forward_triples(triples).view(B, R)
            if return_indices:
                s, idx = torch.topk(batch_scores, topk, dim=1)
                scores[i:i + batch_size, :] = s.cpu()
                indices[i:i + batch_size, :] = idx.cpu()
            else:
                scores[i * R:i * R + B * R] = batch_scores.flatten().cpu()
        if return_indices:
            return scores.flatten(), indices.flatten()
        return scores

    def predict(self, *, h: Union[List[str], str] = None, r: Union[List[str], str] = None,
                t: Union[List[str], str] = None, within=None, logits=True) -> torch.FloatTensor:
        if h is not None:
            assert isinstance(h, (list, str))
        if r is not None:
            assert isinstance(r, (list, str))
        if t is not None:
            assert isinstance(t, (list, str))
        if h is None:
            assert r is not None and t is not None
            scores = self.predict_missing_head_entity(r, t, within)
        elif r is None:
            assert h is not None and t is not None
            scores = self.predict_missing_relations(h, t, within)
        elif t is None:
            scores = self.predict_missing_tail_entity(h, r, within)
        else:
            scores = self.triple_score(h, r, t, logits=True).cpu()
        return scores if logits else torch.sigmoid(scores)

    def triple_score(self, h: Union[List[str], str] = None, r: Union[List[str], str] = None,
                     t: Union[List[str], str] = None, logits=False) -> torch.FloatTensor:
        """Score (sigmoid unless ``logits``) of the given triples; lists are taken element-wise (:581-650)."""
        if isinstance(h, list) and isinstance(r, list) and isinstance(t, list):
            hh = [self.entity_to_idx[i] for i in h]
            rr = [self.relation_to_idx[i] for i in r]
            tt = [self.entity_to_idx[i] for i in t]
        else:
            hh, rr, tt = [self.entity_to_idx[h]], [self.relation_to_idx[r]], [self.entity_to_idx[t]]
        x = torch.stack([torch.LongTensor(hh), torch.LongTensor(rr), torch.LongTensor(tt)], dim=1)
        with torch.no_grad():
            s = self.model(x.to(self.model.entity_embeddings.weight.device))
        return s if logits else torch.sigmoid(s)

    def predict_topk(self, *, h: Union[str, List[str]] = None, r: Union[str, List[str]] = None,
                     t: Union[str, List[str]] = None, topk: int = 10, within: List[str] = None,
                     batch_size: int = 1024):
        """``List[P] of List[topk] of (entity, sigmoid(score))`` for the P = len(h)*len(r) queries."""
        if h is not None:
            assert isinstance(h, (list, str))
        if r is not None:
            assert isinstance(r, (list, str))
        if t is not None:
            assert isinstance(t, (list, str))
        if h is None:
            assert r is not None and t is not None
            r = [r] if isinstance(r, str) else r
            t = [t] if isinstance(t, str) else t
            flat_scores, flat_indices = self.predict_missing_head_entity(r, t, within, batch_size, topk,
                                                                         return_indices=True)
            num_hr_pairs = len(r) * len(t)
        elif r is None:
            assert h is not None and t is not None
            flat_scores, flat_indices = self.predict_missing_relations(h, t, within, batch_size, topk,
                                                                       return_indices=True)
            h = [h] if isinstance(h, str) else h
            t = [t] if isinstance(t, str) else t
            num_hr_pairs = len(h) * len(t)
            scores_2d = flat_scores.view(num_hr_pairs, topk)
            indices_2d = flat_indices.view(num_hr_pairs, topk)
            return [[(self.idx_to_relations[idx], score) for idx, score in zip(row_idxs, row_scores)]
                    for row_idxs, row_scores in zip(indices_2d.tolist(), torch.sigmoid(scores_2d).tolist())]
        elif t is not None:
            raise AttributeError("Use triple_score method")
        else:
            flat_scores, flat_indices = self.predict_missing_tail_entity(h, r, within, batch_size, topk,
                                                                         return_indices=True)
            h = [h] if isinstance(h, str) else h
            r = [r] if isinstance(r, str) else r
            num_hr_pairs = len(h) * len(r)
        scores_2d = flat_scores.view(num_hr_pairs, topk)
        indices_2d = flat_indices.view(num_hr_pairs, topk)
        topk_scores = torch.sigmoid(scores_2d).tolist()
        topk_idxs = indices_2d.tolist()
        lookup = self.idx_to_entity
        return [[(lookup[idx], score) for idx, score in zip(row_idxs, row_scores)]
                for row_idxs, row_scores in zip(topk_idxs, topk_scores)]

    # ------------------------------------------------------------------ multi-hop queries
    @staticmethod
    def t_norm(tens_1, tens_2, tnorm="min"):
        """dicee/abstracts.py:443-447."""
        if "min" in tnorm:
            return torch.min(tens_1, tens_2)
        if "prod" in tnorm:
            return tens_1 * tens_2

    @staticmethod
    def t_conorm(tens_1, tens_2, tconorm="min"):
        """dicee/abstracts.py:460-464."""
        if "min" in tconorm:
            return torch.max(tens_1, tens_2)
        if "prod" in tconorm:
            return (tens_1 + tens_2) - (tens_1 * tens_2)

    @staticmethod
    def negnorm(tens_1, lambda_, neg_norm="standard"):
        """dicee/abstracts.py:466-472."""
        if "standard" in neg_norm:
            return 1 - tens_1
        if "sugeno" in neg_norm:
            return (1 - tens_1) / (1 + lambda_ * tens_1)
        if "yager" in neg_norm:
            return (1 - torch.pow(tens_1, lambda_)) ** (1 / lambda_)

    def _atom(self, head_ids, relation: str):
        """[len(head_ids), N] logits of (head, relation, ?) on the GPU: ONE batched KvsAll call where the
        reference calls ``predict`` once per substitution."""
        dev = self.model.entity_embeddings.weight.device
        head_ids = torch.as_tensor(head_ids, dtype=torch.int64, device=dev).reshape(-1)
        rel = torch.full_like(head_ids, self.relation_to_idx[relation])
        with torch.no_grad():
            return self.model.forward_k_vs_all(torch.stack([head_ids, rel], dim=1).contiguous())

    def _multi_hop_scores(self, query_type, query, tnorm, neg_norm, lambda_, k):
        """[N] GPU tensor: score of every entity as the answer (the norms act on logits, as in the reference,
        whose ``predict`` defaults to ``logits=True``)."""
        one = lambda e, r: self._atom([self.entity_to_idx[e]], r)[0]

        def hop(prev, r):          # keep the k best substitutions of the variable, then the best t-norm per answer
            s, idx = torch.sort(prev, descending=True, stable=True)
            return torch.max(self.t_norm(s[:k, None], self._atom(idx[:k], r), tnorm), dim=0)[0]
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
            vals = []
            for e, rel in (part for part in query if part != ("u",)):
                v = one(e, rel[0])
                vals.append(self.negnorm(v, lambda_, neg_norm) if rel[-1] == "n" else v)
            out = vals[0]
            for v in vals[1:]:
                out = self.t_conorm(out, v, tnorm) if query_type == "2u" else self.t_norm(out, v, tnorm)
            return out
        if query_type in ("ip", "inp", "up"):
            inner, (r,) = query
            inner_type = {"ip": "2i", "inp": "2in", "up": "2u"}[query_type]
            return hop(self._multi_hop_scores(inner_type, inner, tnorm, neg_norm, lambda_, k), r)
        if query_type in ("pi", "pin", "pni"):
            (e1, rels), (e3, rel3) = query
            s, idx = torch.sort(one(e1, rels[0]), descending=True, stable=True)
            a2 = self._atom(idx[:k], rels[1])
            if query_type == "pni":
                a2 = self.negnorm(a2, lambda_, neg_norm)
            two_p = torch.max(self.t_norm(s[:k, None], a2, tnorm), dim=0)[0]
            last = one(e3, rel3[0])
            if query_type == "pin":
                last = self.negnorm(last, lambda_, neg_norm)
            return self.t_norm(two_p, last, tnorm)
        raise ValueError(f"Invalid query type: {query_type}")

    def answer_multi_hop_query(self, query_type: str = None, query=None, queries=None, tnorm: str = "prod",
                               neg_norm: str = "standard", lambda_: float = 0.0, k: int = 10, only_scores=False):
        """Answers of an EPFO query with negation and disjunction (types 1p 2p 3p 2i 3i ip pi 2in 3in inp pin pni
        2u up; query encodings as in the reference, e.g. 2p = ``(e, (r1, r2))``, 2i = ``((e1, (r1,)), (e2, (r2,)))``).
        ``only_scores``: the [N] score tensor; else ``[(entity, score), ...]`` sorted by score, the best k for the
        path types 1p / 2p / 3p and all entities for the others."""
        if queries is not None:
            assert query is None
            return [self.answer_multi_hop_query(query_type=query_type, query=q, tnorm=tnorm, neg_norm=neg_norm,
                                                lambda_=lambda_, k=k, only_scores=only_scores) for q in queries]
        assert len(self.entity_to_idx) >= k >= 0
        scores = self._multi_hop_scores(query_type, query, tnorm, neg_norm, lambda_, k).cpu()
        if only_scores:
            return scores
        order = torch.sort(scores, descending=True, stable=True)[1].tolist()
        if query_type in ("1p", "2p", "3p"):
            order = order[:k]
        return [(self.idx_to_entity[i], scores[i]) for i in order]
