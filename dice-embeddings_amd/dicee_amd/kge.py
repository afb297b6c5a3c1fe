"""Interactive tail prediction on top of the fused top-k kernel.

Mirrors the tail branch of dicee's ``KGE`` (dicee/knowledge_graph_embeddings.py):
``predict_missing_tail_entity`` (:314-413), ``predict`` (:415-466) and ``predict_topk`` (:468-579).
Head and relation prediction go through ``forward_triples`` in the reference and are outside this
build: they raise ``NotImplementedError``.
"""
from typing import List, Union

import torch


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

    def predict(self, *, h: Union[List[str], str] = None, r: Union[List[str], str] = None,
                t: Union[List[str], str] = None, within=None, logits=True) -> torch.FloatTensor:
        if h is not None:
            assert isinstance(h, (list, str))
        if r is not None:
            assert isinstance(r, (list, str))
        if t is not None:
            assert isinstance(t, (list, str))
        if t is None:
            assert h is not None and r is not None
            scores = self.predict_missing_tail_entity(h, r, within)
        elif h is None or r is None:
            raise NotImplementedError("head / relation prediction is outside the accelerated path")
        else:
            raise NotImplementedError("triple_score is outside the accelerated path")
        return scores if logits else torch.sigmoid(scores)

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
        if h is None or r is None:
            raise NotImplementedError("head / relation prediction is outside the accelerated path")
        if t is not None:
            raise AttributeError("Use triple_score method")
        flat_scores, flat_indices = self.predict_missing_tail_entity(h, r, within, batch_size, topk,
                                                                     return_indices=True)
        if isinstance(h, str):
            h = [h]
        if isinstance(r, str):
            r = [r]
        num_hr_pairs = len(h) * len(r)
        scores_2d = flat_scores.view(num_hr_pairs, topk)
        indices_2d = flat_indices.view(num_hr_pairs, topk)
        topk_scores = torch.sigmoid(scores_2d).tolist()
        topk_idxs = indices_2d.tolist()
        lookup = self.idx_to_entity
        return [[(lookup[idx], score) for idx, score in zip(row_idxs, row_scores)]
                for row_idxs, row_scores in zip(topk_idxs, topk_scores)]
