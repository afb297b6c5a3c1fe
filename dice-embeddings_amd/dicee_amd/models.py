"""Model containers with the reference's KvsAll call surface, backed by the HIP kernels.

Parameter names follow dicee so that a dicee ``model.pt`` state_dict loads unchanged
(``entity_embeddings.weight``, ``relation_embeddings.weight``, Keci's ``p_coefficients.weight`` /
``q_coefficients.weight``, ``normalize_*_embeddings.*``): dicee/models/base_model.py:121-176,
dicee/models/clifford.py:4-28.

Layers follow the module's mode.  LayerNorm is the same in both; BatchNorm1d normalises with its running
statistics in eval mode and with the statistics of the batch in training mode (moving the running statistics, as
torch does).  Dropout (base_model.py:149-151) is the identity in eval mode; in training mode with
``input_dropout_rate`` > 0 the looked-up head and relation rows, and DistMult's ``h * r``, are dropped element by
element with masks drawn from torch's generator on the device (the distribution of torch.nn.Dropout, not its
stream: no two implementations share that).
"""
import torch

from . import ops


class IdentityClass(torch.nn.Module):
    """dicee/models/base_model.py:441-450; QMult also uses it as a type test (quaternion.py:138)."""

    def __init__(self, args=None):
        super().__init__()
        self.args = args

    @staticmethod
    def forward(x):
        return x


_FROM_MODEL = object()   # "take the normalisation layer from the model" (None means: no layer)


class BaseKGE(torch.nn.Module):
    name = "BaseKGE"

    def __init__(self, args: dict):
        super().__init__()
        self.args = dict(args)
        self.embedding_dim = int(args["embedding_dim"])
        self.num_entities = int(args["num_entities"])
        self.num_relations = int(args["num_relations"])
        self.input_dropout_rate = float(args.get("input_dropout_rate", 0.0) or 0.0)
        self.hidden_dropout_rate = float(args.get("hidden_dropout_rate", 0.0) or 0.0)
        self.loss = torch.nn.BCEWithLogitsLoss()
        self.normalize_head_entity_embeddings = IdentityClass()
        self.normalize_relation_embeddings = IdentityClass()
        self.normalize_tail_entity_embeddings = IdentityClass()
        self.hidden_normalizer = IdentityClass()
        norm = args.get("normalization")
        # a model trained on single triples also normalises the tail row (base_model.py:287-294); KvsAll scoring
        # never does (the table is used as it is), only forward_triples
        tail_too = args.get("scoring_technique") in ("NegSample", "KvsSample")
        if norm == "LayerNorm":
            self.normalize_head_entity_embeddings = torch.nn.LayerNorm(self.embedding_dim)
            self.normalize_relation_embeddings = torch.nn.LayerNorm(self.embedding_dim)
            if tail_too:
                self.normalize_tail_entity_embeddings = torch.nn.LayerNorm(self.embedding_dim)
        elif norm == "BatchNorm1d":
            self.normalize_head_entity_embeddings = torch.nn.BatchNorm1d(self.embedding_dim, affine=False)
            self.normalize_relation_embeddings = torch.nn.BatchNorm1d(self.embedding_dim, affine=False)
            if tail_too:
                self.normalize_tail_entity_embeddings = torch.nn.BatchNorm1d(self.embedding_dim, affine=False)
        elif norm is not None:
            raise NotImplementedError(norm)
        self.entity_embeddings = torch.nn.Embedding(self.num_entities, self.embedding_dim)
        self.relation_embeddings = torch.nn.Embedding(self.num_relations, self.embedding_dim)
        self._storage = "fp32"
        self._table = None       # quantised / bf16 copy of the entity table
        self._scale = None
        self._rel_table = None
        self._snap_key = None    # identity and version of the parameters the bf16 / int8 copies were taken from
        self._topk_prepared = None   # (table data_ptr, derived form of the table that top-k scans), made on first use

    # ------------------------------------------------------------------ storage
    def set_entity_storage(self, kind="fp32"):
        """Keep the tables the kernels read as ``fp32`` (the parameters themselves), ``bf16``
        (entities and relations rounded to bf16) or ``int8`` (entities per-row symmetric int8 with
        an fp32 scale per row, relations fp32).  Scores then follow fp32 math on the dequantised
        table."""
        w = self.entity_embeddings.weight.detach()
        if kind == "fp32":
            self._table = self._scale = self._rel_table = None
        elif kind == "bf16":
            self._table = w.to(torch.bfloat16).contiguous()
            self._scale = None
            self._rel_table = self.relation_embeddings.weight.detach().to(torch.bfloat16).contiguous()
        elif kind == "int8":
            amax = w.abs().amax(dim=1)
            scale = (amax / 127.0).to(torch.float32)
            safe = torch.where(scale > 0, scale, torch.ones_like(scale))
            self._table = torch.round(w / safe[:, None]).clamp(-127, 127).to(torch.int8).contiguous()
            self._scale = scale.contiguous()
            self._rel_table = None
        else:
            raise ValueError(kind)
        self._storage = kind
        self._snap_key = self._parameter_key()
        self._topk_prepared = None
        return self

    def _parameter_key(self):
        we, wr = self.entity_embeddings.weight, self.relation_embeddings.weight
        return (we.data_ptr(), we._version, wr.data_ptr(), wr._version)

    def _refresh_storage(self):
        """The bf16 / int8 tables are copies: take them again when the parameters have changed since (an
        optimizer step, ``load_state_dict``, a move to another device).  The change is seen through the parameters'
        storage address and autograd version counter, which in-place writes THROUGH ``weight.data`` do not advance
        (``param_init(self.entity_embeddings.weight.data)`` in the reference, ``weight.data.copy_(...)`` in user
        code): after such a write call ``refresh_storage()``."""
        if self._storage != "fp32" and self._snap_key != self._parameter_key():
            self.set_entity_storage(self._storage)

    def refresh_storage(self):
        """Take the bf16 / int8 copies of the tables (and the int8 table's prepared form for top-k) again from the
        parameters as they are now.  Needed only after in-place writes through ``weight.data``, which leave no
        trace the model could see; every other change of the parameters is picked up by itself."""
        if self._storage != "fp32":
            self.set_entity_storage(self._storage)
        return self

    def table(self):
        """(entity table the kernels read, per-row scale or None)."""
        self._refresh_storage()
        if self._table is not None:
            return self._table, self._scale
        return self.entity_embeddings.weight.detach(), None

    def _rel(self):
        self._refresh_storage()
        return self._rel_table if self._rel_table is not None else self.relation_embeddings.weight.detach()

    def _draw_dropout(self, B, device, rows=True):
        """The masks one training-mode forward over B pairs applies: ``input_dp_ent_real`` on the head rows and
        ``input_dp_rel_real`` on the relation rows (base_model.py:381-383), and for DistMult ``hidden_dropout`` on
        ``h * r`` (real.py:32), all three built with ``input_dropout_rate`` (base_model.py:149-151; the models of this
        path never read ``hidden_dropout_rate``).  None in eval mode or with a rate of zero."""
        rate = self.input_dropout_rate
        if not self.training or rate <= 0.0:
            return None
        if rate >= 1.0:
            raise ValueError("a dropout rate of 1 leaves nothing")
        d = self.embedding_dim
        drop = {"scale_in": 1.0 / (1.0 - rate), "scale_hidden": 1.0 / (1.0 - rate)}
        if rows:
            drop["keep_h"] = (torch.rand((B, d), device=device) >= rate).to(torch.uint8)
            drop["keep_r"] = (torch.rand((B, d), device=device) >= rate).to(torch.uint8)
        if self.name == "DistMult":
            drop["keep_q"] = (torch.rand((B, d), device=device) >= rate).to(torch.uint8)
        return drop if len(drop) > 2 else None

    # ------------------------------------------------------------------ query construction
    def _norm_params(self, x=None, dropout=None):
        """The normalisation layer between the lookups and the interaction, as the kernels take it.  BatchNorm1d in
        training mode normalises with the statistics of the batch ``x`` [B,2] itself and moves its running
        statistics towards them (torch.nn.BatchNorm1d; base_model.py:289-294 applied at :381-383): every call with
        a batch is one such forward.  ``dropout``: the masks of this forward (the layer sees the rows after dropout)."""
        nh, nr = self.normalize_head_entity_embeddings, self.normalize_relation_embeddings
        if isinstance(nh, torch.nn.LayerNorm):
            return {"kind": "LayerNorm", "eps": nh.eps, "h_a": nh.weight.detach(), "h_b": nh.bias.detach(),
                    "r_a": nr.weight.detach(), "r_b": nr.bias.detach()}
        if isinstance(nh, torch.nn.BatchNorm1d):
            if self.training and x is not None:
                if self._storage != "fp32":
                    raise NotImplementedError("BatchNorm1d in training mode needs the fp32 tables")
                if nh.momentum is None or nr.momentum is None or nh.momentum != nr.momentum:
                    raise NotImplementedError("BatchNorm1d with a cumulative average (momentum=None) or two momenta")
                E, _ = self.table()
                pairs = x.to(device=E.device, dtype=torch.int64).contiguous()
                running = None
                if nh.track_running_stats and nh.running_mean is not None:
                    running = {"h_mean": nh.running_mean, "h_var": nh.running_var, "r_mean": nr.running_mean,
                               "r_var": nr.running_var}
                norm = ops.batchnorm_stats(E, self._rel(), pairs, eps=nh.eps, momentum=nh.momentum, running=running,
                                           dropout=dropout)
                if running is not None:
                    nh.num_batches_tracked += 1
                    nr.num_batches_tracked += 1
                return norm
            return {"kind": "BatchNorm1d", "eps": nh.eps, "h_a": nh.running_mean, "h_b": nh.running_var,
                    "r_a": nr.running_mean, "r_b": nr.running_var}
        return None

    def _query_kwargs(self):
        return {}

    def query(self, x, heads=False, norm=_FROM_MODEL, dropout=_FROM_MODEL):
        """(Q [B,d], bias [B]) for ``x`` [B,2]: gather + interaction
        (get_head_relation_representation, base_model.py:377-384, then the model's elementwise part).
        ``heads=True``: ``x`` holds (relation, tail) pairs and ``Q @ E^T`` scores every entity as the head of
        (x, r, t): what ``forward_triples`` gives triple by triple (base_model.py:346-362)."""
        E, scale = self.table()
        x = x.to(device=E.device, dtype=torch.int64).contiguous()
        if dropout is _FROM_MODEL:
            dropout = self._draw_dropout(x.shape[0], E.device)
        if heads and dropout is not None:
            raise NotImplementedError("head-direction queries in training mode with dropout are not part of this path")
        if norm is _FROM_MODEL:
            norm = self._norm_params(None if heads else x, dropout)
        return ops.build_query(self.name if self.name != "CKeci" else "Keci", E, self._rel(), x, ent_scale=scale,
                               norm=norm, head=heads, dropout=dropout, **self._query_kwargs())

    # ------------------------------------------------------------------ reference call surface
    def forward(self, x, y_idx=None):
        """Shape dispatch of BaseKGE.forward (base_model.py:310-344): [B,2] -> KvsAll scores, [n,3] -> triple scores."""
        if isinstance(x, tuple):
            x, y_idx = x
            return self.forward_k_vs_sample(x=x, target_entity_idx=y_idx)
        if x.dim() == 2 and x.shape[1] == 2:
            return self.forward_k_vs_all(x=x)
        if x.dim() == 2 and x.shape[1] == 3:
            return self.forward_triples(x)
        raise NotImplementedError("byte-pair-encoded inputs are outside the accelerated path")

    def forward_k_vs_all(self, x):
        """[B,N] fp32 scores of every entity as tail; the caller owns (and may mutate) the result."""
        Q, bias = self.query(x)
        E, scale = self.table()
        return ops.scores(Q, bias, E, scale)

    def forward_k_vs_sample(self, x, target_entity_idx):
        """[B,k] fp32 scores of the k entities ``target_entity_idx[b]`` as tails of ``x[b]`` (real.py:38-45 and its
        siblings): the query of (h, r) against the sampled rows only, the same bits as those columns of the KvsAll
        scores."""
        E, scale = self.table()
        Q, bias = self.query(x)
        idx = target_entity_idx.to(device=E.device, dtype=torch.int64)
        return ops.sample_scores(Q, bias, E, scale, idx)

    def forward_triples(self, x):
        """[n] fp32 scores of the triples ``x`` [n,3] = (h, r, t) (base_model.py:346-362): the query of (h, r)
        against the one row E[t], with the reduction order of the KvsAll kernels."""
        E, scale = self.table()
        x = x.to(device=E.device, dtype=torch.int64)
        Q, bias = self.query(x[:, :2].contiguous())
        nt = self.normalize_tail_entity_embeddings
        if isinstance(nt, IdentityClass):
            return ops.triple_scores(Q, bias, E, scale, x[:, 2].contiguous())
        # normalised tails (base_model.py:374) are not rows of the table: the reference's own normaliser module, with
        # eval semantics, makes the n rows, and triple i is scored against row i of that small table
        if self.training:
            raise NotImplementedError("tail normalisation in training mode (batch statistics) is not part of this path")
        w = self.entity_embeddings.weight.detach()
        idx = x[:, 2].contiguous()
        if (idx < 0).any() or (idx >= self.num_entities).any():
            raise IndexError("index out of range in self")
        with torch.no_grad():
            tails = nt(w[idx]).contiguous().float()
        return ops.triple_scores(Q, bias, tails, None, torch.arange(idx.numel(), device=E.device, dtype=torch.int64))

    def forward_all_heads(self, rt):
        """[B,N] fp32: score(x, r, t) of every entity x as head, for ``rt`` [B,2] = (relation, tail) pairs."""
        Q, bias = self.query(rt, heads=True)
        E, scale = self.table()
        return ops.scores(Q, bias, E, scale)

    def k_vs_all_score(self, emb_h, emb_r, emb_E):
        """Scores from already gathered rows: [B,d],[B,d],[N,d] -> [B,N] (in training mode DistMult drops elements of
        ``h * r`` here, real.py:32; the rows themselves are the caller's)."""
        B = emb_h.shape[0]
        idx = torch.arange(B, device=emb_h.device, dtype=torch.int64)
        hr = torch.stack([idx, idx], dim=1).contiguous()
        Q, bias = ops.build_query(self.name if self.name != "CKeci" else "Keci", emb_h.contiguous().float(),
                                  emb_r.contiguous().float(), hr, dropout=self._draw_dropout(B, emb_h.device, rows=False),
                                  **self._query_kwargs())
        return ops.scores(Q, bias, emb_E.contiguous().float())

    def get_embeddings(self):
        """(entity embeddings, relation embeddings), detached tensors as the reference returns them
        (base_model.py:431-438; its annotation says ndarray, its code returns tensors)."""
        return self.entity_embeddings.weight.detach(), self.relation_embeddings.weight.detach()

    # ------------------------------------------------------------------ fused consumers
    def rank_filtered(self, x, target, csr=None, heads=False, out=None):
        """Fused filtered-rank counters for queries ``x`` [B,2] and true tails ``target`` [B].
        ``heads=True``: ``x`` = (relation, tail) pairs, ``target`` the true heads, ``csr`` the (r, t) -> heads
        vocabulary.  ``out``: the dict of [B] tensors to write into (``ops.rank_filtered``)."""
        Q, bias = self.query(x, heads=heads)
        E, scale = self.table()
        target = target.to(device=E.device, dtype=torch.int64).contiguous()
        if csr is None:
            return ops.rank_filtered(Q, bias, E, scale, target, out=out)
        rows = csr.rows_for(x.to(device=E.device, dtype=torch.int64))
        return ops.rank_filtered(Q, bias, E, scale, target, rows, csr.row_ptr, csr.col, out=out)

    def topk(self, x, k, sigmoid=False, heads=False):
        Q, bias = self.query(x, heads=heads)
        E, scale = self.table()
        # the quantised table's derived form for the scan lives and dies with the quantised table itself
        prepared = None
        if self._table is not None and scale is not None:
            if self._topk_prepared is None or self._topk_prepared[0] != E.data_ptr():
                self._topk_prepared = (E.data_ptr(), ops.topk_prepare(E, scale))
            prepared = self._topk_prepared[1]
        return ops.topk(Q, bias, E, scale, k, sigmoid=sigmoid, prepared=prepared)

    def kvsall_bce_loss(self, x, csr, label_smoothing=0.0):
        """Forward + loss of training_step (base_model.py:25-46) for a KvsAll batch whose multi-hot
        target is given by the CSR rows of ``x`` (dataset_classes.py:354-361)."""
        Q, bias = self.query(x)
        E, scale = self.table()
        rows = csr.rows_for(x.to(device=E.device, dtype=torch.int64))
        return ops.bce_multihot(Q, bias, E, scale, rows, csr.row_ptr, csr.col, label_smoothing)[0]

    def kvsall_bce_backward(self, x, csr, label_smoothing=0.0, grad_out=1.0, norm=_FROM_MODEL, dropout=_FROM_MODEL):
        """The same step with its backward through the scores: ``(loss, dQ [B,d], dbias [B], dE [N,d])`` where
        ``dQ`` / ``dbias`` are the gradients at the query vectors and per-query biases of ``self.query(x)`` and ``dE``
        the gradient the contraction sends to the entity table (fp32 tables only).  What
        ``loss_batch.backward()`` computes for the ``torch.mm`` / ``einsum`` and the loss of the reference's step."""
        Q, bias = self.query(x, norm=norm, dropout=dropout)
        E, scale = self.table()
        if scale is not None:
            raise TypeError("the backward needs an fp32 entity table")
        rows = csr.rows_for(x.to(device=E.device, dtype=torch.int64))
        loss, dQ, dbias, dE = ops.bce_multihot_backward(Q, bias, E, rows, csr.row_ptr, csr.col, label_smoothing, grad_out)
        return loss[0], dQ, dbias, dE

    def kvsall_bce_gradients(self, x, csr, label_smoothing=0.0):
        """Loss of the KvsAll BCE step and its gradient at every parameter the step reads:
        ``(loss, {parameter name: gradient})`` with ``entity_embeddings.weight`` [N,d] (the contraction's gradient
        plus the rows of the heads), ``relation_embeddings.weight`` [R,d] and, for Keci / DeCaL, the coefficient
        embeddings.  What ``loss_batch.backward()`` leaves in ``.grad`` after ``training_step`` (base_model.py:25-46)
        for fp32 tables.  With ``normalization='LayerNorm'`` the gradient passes through both normalisers and their
        weights and biases receive theirs (``normalize_head_entity_embeddings.weight`` ...); with ``'BatchNorm1d'``
        it passes through the statistics of the batch in training mode (which also moves the running statistics, once)
        and through the running statistics in eval mode.  In training mode with ``input_dropout_rate`` > 0 one set of
        masks is drawn for the step and used by its forward and its backward."""
        E, scale = self.table()
        if scale is not None or E.dtype != torch.float32:
            raise TypeError("the backward needs an fp32 entity table")
        x = x.to(device=E.device, dtype=torch.int64).contiguous()
        dropout = self._draw_dropout(x.shape[0], E.device)
        norm = self._norm_params(x, dropout)
        loss, dQ, dbias, dE = self.kvsall_bce_backward(x, csr, label_smoothing, norm=norm, dropout=dropout)
        rel = self._rel()
        dR = torch.zeros_like(rel)
        name = self.name if self.name != "CKeci" else "Keci"
        dnorm = None
        if norm is not None and norm["kind"] == "LayerNorm":
            dnorm = {k: torch.zeros_like(norm[k], dtype=torch.float32) for k in ("h_a", "h_b", "r_a", "r_b")}
        dcoeff = ops.build_query_backward(name, E, rel, x, dQ, dbias, dE, dR, norm=norm, dnorm=dnorm, dropout=dropout,
                                          **self._query_kwargs())
        grads = {"entity_embeddings.weight": dE, "relation_embeddings.weight": dR}
        if dnorm is not None:
            grads["normalize_head_entity_embeddings.weight"] = dnorm["h_a"]
            grads["normalize_head_entity_embeddings.bias"] = dnorm["h_b"]
            grads["normalize_relation_embeddings.weight"] = dnorm["r_a"]
            grads["normalize_relation_embeddings.bias"] = dnorm["r_b"]
        for key, g in zip(("p_coefficients.weight", "q_coefficients.weight", "r_coefficients.weight"), dcoeff):
            if g is not None:
                grads[key] = g.reshape(1, -1)
        return loss, grads

    def kvsall_training_step(self, x, csr, label_smoothing=0.0):
        """``training_step`` followed by ``loss.backward()`` (base_model.py:25-46) for one KvsAll batch: returns the
        loss (detached) and ACCUMULATES the gradients into ``.grad`` of the parameters the step reads, as
        autograd would, so that any ``torch.optim`` optimizer can take the step."""
        loss, grads = self.kvsall_bce_gradients(x, csr, label_smoothing)
        params = dict(self.named_parameters())
        for name, g in grads.items():
            prm = params[name]
            if not prm.requires_grad:
                continue
            prm.grad = g if prm.grad is None else prm.grad + g
        return loss


class DistMult(BaseKGE):
    """dicee/models/real.py:10-36."""
    name = "DistMult"


class ComplEx(BaseKGE):
    """dicee/models/complex.py:223-269."""
    name = "ComplEx"


class QMult(BaseKGE):
    """dicee/models/quaternion.py:24-171."""
    name = "QMult"

    def _query_kwargs(self):
        # the quaternion normaliser runs only when no other relation normaliser is set (quaternion.py:138)
        return {"normalize_relation": isinstance(self.normalize_relation_embeddings, IdentityClass)}


class OMult(BaseKGE):
    """dicee/models/octonion.py:51-163."""
    name = "OMult"

    def __init__(self, args):
        super().__init__(args)
        assert self.embedding_dim % 8 == 0, "OMult needs an embedding dimension divisible by 8"

    def _query_kwargs(self):
        # the octonion normaliser runs only when no other relation normaliser is set (octonion.py:121)
        return {"normalize_relation": isinstance(self.normalize_relation_embeddings, IdentityClass)}


class Keci(BaseKGE):
    """dicee/models/clifford.py:3-329."""
    name = "Keci"

    def __init__(self, args):
        super().__init__(args)
        self.p = int(args.get("p", 0) or 0)
        self.q = int(args.get("q", 0) or 0)
        r = self.embedding_dim / (self.p + self.q + 1)
        if not float(r).is_integer():
            raise AssertionError(f"r = embedding_dim / (p + q+ 1) must be a whole number\n"
                                 f"Currently {r}={self.embedding_dim} / ({self.p}+ {self.q} +1)")
        self.r = int(r)
        if self.p > 0:
            self.p_coefficients = torch.nn.Embedding(num_embeddings=1, embedding_dim=self.p)
            torch.nn.init.zeros_(self.p_coefficients.weight)
        if self.q > 0:
            self.q_coefficients = torch.nn.Embedding(num_embeddings=1, embedding_dim=self.q)
            torch.nn.init.zeros_(self.q_coefficients.weight)

    def _query_kwargs(self):
        kw = {"p": self.p, "q": self.q}
        if self.p > 0:
            kw["coeff_p"] = self.p_coefficients.weight.detach().reshape(-1).float().contiguous()
        if self.q > 0:
            kw["coeff_q"] = self.q_coefficients.weight.detach().reshape(-1).float().contiguous()
        return kw


class CKeci(Keci):
    """Keci without learned dimension scaling (clifford.py:563-576)."""
    name = "CKeci"

    def __init__(self, args):
        super().__init__(args)
        if self.p > 0:
            torch.nn.init.ones_(self.p_coefficients.weight)
            self.p_coefficients.weight.requires_grad_(False)
        if self.q > 0:
            torch.nn.init.ones_(self.q_coefficients.weight)
            self.q_coefficients.weight.requires_grad_(False)


class DeCaL(BaseKGE):
    """dicee/models/clifford.py:579-912: Cl(p, q, r) with r degenerate bases.  Parameter names and shapes as there
    (``p_coefficients`` / ``q_coefficients`` / ``r_coefficients``: Embedding(1, count), zero-initialised); ``re`` is
    the length of one part.  The reference truncates ``embedding_dim / (1 + p + q + r)``; a remainder would leave
    columns that no term reads, so it is refused here."""
    name = "DeCaL"

    def __init__(self, args):
        super().__init__(args)
        self.p = int(args.get("p", 0) or 0)
        self.q = int(args.get("q", 0) or 0)
        self.r = int(args.get("r", 0) or 0)
        parts = self.p + self.q + self.r + 1
        if self.embedding_dim % parts:
            raise AssertionError(f"embedding_dim / (p + q + r + 1) must be a whole number\n"
                                 f"Currently {self.embedding_dim} / ({self.p} + {self.q} + {self.r} + 1)")
        self.re = self.embedding_dim // parts
        for count, attr in ((self.p, "p_coefficients"), (self.q, "q_coefficients"), (self.r, "r_coefficients")):
            if count > 0:
                emb = torch.nn.Embedding(num_embeddings=1, embedding_dim=count)
                torch.nn.init.zeros_(emb.weight)
                setattr(self, attr, emb)

    def _query_kwargs(self):
        kw = {"p": self.p, "q": self.q, "r": self.r}
        for count, attr, key in ((self.p, "p_coefficients", "coeff_p"), (self.q, "q_coefficients", "coeff_q"),
                                 (self.r, "r_coefficients", "coeff_r")):
            if count > 0:
                kw[key] = getattr(self, attr).weight.detach().reshape(-1).float().contiguous()
        return kw


MODEL_REGISTRY = {"DistMult": DistMult, "ComplEx": ComplEx, "QMult": QMult, "OMult": OMult, "Keci": Keci,
                  "CKeci": CKeci, "DeCaL": DeCaL}


def initialize_model(args: dict):
    """(model, 'EntityPrediction') as dicee.static_funcs.intialize_model (static_funcs.py:483-509)."""
    name = args["model"]
    if name not in MODEL_REGISTRY:
        raise ValueError(f"--model_name: {name} is not found.")
    return MODEL_REGISTRY[name](args), "EntityPrediction"
