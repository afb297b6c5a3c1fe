"""Tensor-level wrappers of the C ABI.  torch is used for device memory and streams only."""
import ctypes

import torch

from . import _lib
from ._lib import MODEL_IDS, DTYPE_F32, DTYPE_BF16, DTYPE_I8, NormParams

_TORCH_TO_KGE = {torch.float32: DTYPE_F32, torch.bfloat16: DTYPE_BF16, torch.int8: DTYPE_I8}


def _require_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("dicee_amd ops need tensors on the GPU (there is no CPU path)")
        if not t.is_contiguous():
            raise ValueError("dicee_amd ops need contiguous tensors")


def _check_qe(Q, E, scale=None, bias=None):
    """Shapes the kernels rely on: Q [B,d] fp32 and E [N,d] share d; bias [B]; scale [N]."""
    if Q.dim() != 2 or E.dim() != 2 or Q.shape[1] != E.shape[1]:
        raise ValueError(f"Q {tuple(Q.shape)} and E {tuple(E.shape)} must be [B,d] and [N,d] with the same d")
    if Q.dtype != torch.float32:
        raise TypeError("Q must be float32")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != Q.shape[0]):
        raise ValueError("bias must be float32 [B]")
    if scale is not None and (scale.dtype != torch.float32 or scale.numel() != E.shape[0]):
        raise ValueError("scale must be float32 [N]")
    if E.dtype == torch.int8 and scale is None:
        raise ValueError("int8 tables need per-row scales")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream of the current device as a ``hipStream_t``.  (torch's C accessor where it has one: building a
    ``torch.cuda.Stream`` object per call costs about as much host time as the rest of a call's issue.)"""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _table_dtype(E):
    try:
        return _TORCH_TO_KGE[E.dtype]
    except KeyError:
        raise TypeError(f"unsupported table dtype {E.dtype}; use float32, bfloat16 or int8") from None


def _norm_struct(norm):
    """norm: None or dict(kind='LayerNorm'|'BatchNorm1d', h_a, h_b, r_a, r_b, eps) of fp32 GPU tensors."""
    if norm is None:
        return None, ()
    kind = {"LayerNorm": _lib.NORM_LAYERNORM, "BatchNorm1d": _lib.NORM_BATCHNORM1D}[norm["kind"]]
    keep = tuple(norm[k].contiguous().float() for k in ("h_a", "h_b", "r_a", "r_b"))
    _require_gpu(*keep)
    s = NormParams(kind, float(norm.get("eps", 1e-5)), *[t.data_ptr() for t in keep])
    return s, keep


def _dropout_struct(dropout, B, d):
    """dropout: None or dict with any of ``keep_h, keep_r, keep_q`` ([B,d] uint8 / bool GPU tensors, nonzero = keep)
    and ``scale_in`` / ``scale_hidden`` (1 / (1 - rate))."""
    if dropout is None:
        return None, ()
    keep = []
    for k in ("keep_h", "keep_r", "keep_q"):
        t = dropout.get(k)
        if t is not None:
            if t.dtype == torch.bool:
                t = t.to(torch.uint8)
            if t.dtype != torch.uint8 or tuple(t.shape) != (B, d):
                raise TypeError(f"dropout mask {k} must be a [B, d] uint8 or bool tensor")
            t = t.contiguous()
            _require_gpu(t)
        keep.append(t)
    s = _lib.DropoutParams(*[t.data_ptr() if t is not None else None for t in keep],
                           float(dropout.get("scale_in", 1.0)), float(dropout.get("scale_hidden", 1.0)))
    return s, tuple(keep)


def build_query(model, ent, rel, hr, *, ent_scale=None, p=0, q=0, r=0, coeff_p=None, coeff_q=None, coeff_r=None,
                normalize_relation=True, norm=None, head=False, dropout=None):
    """(Q [B,d] fp32, bias [B] fp32) with ``forward_k_vs_all(x) == Q @ E^T + bias[:, None]``.
    ``head=True``: ``hr`` holds (relation, tail) pairs and ``Q @ E^T`` scores every entity as the head.
    ``dropout``: the masks of a training-mode forward (``_dropout_struct``)."""
    lib = _lib.load()
    _require_gpu(ent, rel, hr, ent_scale, coeff_p, coeff_q, coeff_r)
    if hr.dtype != torch.int64 or hr.dim() != 2 or hr.shape[1] != 2:
        raise ValueError("hr must be an int64 tensor of shape [B, 2]")
    B, (N, d), R = hr.shape[0], ent.shape, rel.shape[0]
    if rel.shape[1] != d:
        raise ValueError("entity and relation tables must have the same embedding dim")
    Q = torch.empty((B, d), dtype=torch.float32, device=ent.device)
    bias = torch.empty((B,), dtype=torch.float32, device=ent.device)
    ns, keep = _norm_struct(norm)
    if dropout is not None:
        if head:
            raise ValueError("no dropout in the head direction")
        ds, dkeep = _dropout_struct(dropout, B, d)
        rc = lib.kge_build_query_dropout(MODEL_IDS[model], int(p), int(q), int(r), _ptr(ent), _table_dtype(ent),
                                         _ptr(ent_scale), _ptr(rel), _table_dtype(rel), _ptr(coeff_p), _ptr(coeff_q),
                                         _ptr(coeff_r), int(bool(normalize_relation)),
                                         ctypes.byref(ns) if ns is not None else None, ctypes.byref(ds), _ptr(hr), B, d,
                                         N, R, _ptr(Q), _ptr(bias), _stream())
        _lib.check(rc)
        del keep, dkeep
        return Q, bias
    if model == "DeCaL":
        rc = lib.kge_build_query_decal(int(bool(head)), int(p), int(q), int(r), _ptr(ent), _table_dtype(ent),
                                       _ptr(ent_scale), _ptr(rel), _table_dtype(rel), _ptr(coeff_p), _ptr(coeff_q),
                                       _ptr(coeff_r), ctypes.byref(ns) if ns is not None else None, _ptr(hr), B, d, N,
                                       R, _ptr(Q), _ptr(bias), _stream())
        _lib.check(rc)
        del keep
        return Q, bias
    fn = lib.kge_build_query_head if head else lib.kge_build_query
    rc = fn(MODEL_IDS[model], int(p), int(q), _ptr(ent), _table_dtype(ent), _ptr(ent_scale),
            _ptr(rel), _table_dtype(rel), _ptr(coeff_p), _ptr(coeff_q), int(bool(normalize_relation)),
            ctypes.byref(ns) if ns is not None else None, _ptr(hr), B, d, N, R, _ptr(Q), _ptr(bias), _stream())
    _lib.check(rc)
    del keep
    return Q, bias


def batchnorm_stats(ent, rel, hr, *, eps=1e-5, momentum=0.1, running=None, dropout=None):
    """The normalisation layer ``BatchNorm1d(affine=False)`` applies to THIS batch in training mode: a ``norm`` dict
    for ``build_query`` holding the mean and biased variance, per feature, of the looked-up head rows and relation
    rows.  ``running``: dict with ``h_mean, h_var, r_mean, r_var`` ([d] fp32 GPU tensors, the modules' buffers),
    updated in place as torch does in training mode."""
    lib = _lib.load()
    _require_gpu(ent, rel, hr)
    if ent.dtype != torch.float32 or rel.dtype != torch.float32 or not ent.is_contiguous() or not rel.is_contiguous():
        raise TypeError("batchnorm_stats needs contiguous fp32 tables")
    if hr.dtype != torch.int64 or hr.dim() != 2 or hr.shape[1] != 2 or not hr.is_contiguous():
        raise ValueError("hr must be a contiguous int64 tensor of shape [B, 2]")
    B, (N, d), R = hr.shape[0], ent.shape, rel.shape[0]
    if B < 2:
        raise ValueError(f"Expected more than 1 value per channel when training, got input size [{B}, {d}]")
    out = torch.empty((4, d), dtype=torch.float32, device=ent.device)
    run = [None] * 4
    if running is not None:
        run = [running[k] for k in ("h_mean", "h_var", "r_mean", "r_var")]
        for t in run:
            if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != d:
                raise TypeError("running statistics must be contiguous fp32 tensors of d elements")
        _require_gpu(*run)
    ws = torch.empty((4 * d,), dtype=torch.float64, device=ent.device)
    ds, dkeep = _dropout_struct(dropout, B, d)
    rc = lib.kge_batchnorm_stats(_ptr(ent), _ptr(rel), _ptr(hr), B, d, N, R,
                                 ctypes.byref(ds) if ds is not None else None, float(momentum), _ptr(out[0]), _ptr(out[1]),
                                 _ptr(out[2]), _ptr(out[3]), _ptr(run[0]), _ptr(run[1]), _ptr(run[2]), _ptr(run[3]),
                                 _ptr(ws), ws.numel() * 8, _stream())
    _lib.check(rc)
    del dkeep
    return {"kind": "BatchNorm1d", "eps": float(eps), "h_a": out[0], "h_b": out[1], "r_a": out[2], "r_b": out[3],
            "batch": True}


def build_query_backward(model, ent, rel, hr, dQ, dbias, d_ent, d_rel, *, p=0, q=0, r=0, coeff_p=None, coeff_q=None,
                         coeff_r=None, normalize_relation=True, norm=None, dnorm=None, dropout=None):
    """Adds the gradients that ``dQ`` [B,d] / ``dbias`` [B] send back through ``build_query`` into ``d_ent`` [N,d]
    and ``d_rel`` [R,d] (fp32, caller-initialised); returns the gradients of the Clifford coefficients
    ``(d_coeff_p, d_coeff_q, d_coeff_r)`` (None where the model has none).  ``norm``: the normalisation layer of
    ``build_query``; ``dnorm``: for LayerNorm, a dict with any of ``h_a, h_b, r_a, r_b`` ([d] fp32,
    caller-initialised) that receive the gradients of the normalisers' weights and biases.  A ``norm`` that
    ``batchnorm_stats`` made for this batch (``norm["batch"]``) is differentiated as a function of the batch."""
    lib = _lib.load()
    _require_gpu(ent, rel, hr, dQ, dbias, d_ent, d_rel, coeff_p, coeff_q, coeff_r)
    for t in (ent, rel, dQ, d_ent, d_rel):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise TypeError("build_query_backward needs contiguous fp32 tensors")
    B, (N, d), R = hr.shape[0], ent.shape, rel.shape[0]
    outs = [torch.zeros_like(c) if c is not None else None for c in (coeff_p, coeff_q, coeff_r)]
    ds, dkeep = _dropout_struct(dropout, B, d)
    dsp = ctypes.byref(ds) if ds is not None else None
    if norm is not None and norm.get("batch"):
        ns, keep = _norm_struct(norm)
        nbytes = lib.kge_batchnorm_workspace_bytes(B, d)
        ws = torch.empty(((nbytes + 7) // 8,), dtype=torch.float64, device=ent.device)
        rc = lib.kge_build_query_backward_batchnorm(
            MODEL_IDS[model], int(p), int(q), int(r), _ptr(ent), _ptr(rel), _ptr(coeff_p), _ptr(coeff_q), _ptr(coeff_r),
            int(bool(normalize_relation)), ctypes.byref(ns), dsp, _ptr(hr), B, d, N, R, _ptr(dQ), _ptr(dbias), _ptr(d_ent),
            _ptr(d_rel), _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _ptr(ws), ws.numel() * 8, _stream())
        _lib.check(rc)
        del keep
        return tuple(outs)
    if norm is not None or ds is not None:
        ns, keep = _norm_struct(norm)
        gs = None
        if dnorm:
            for t in dnorm.values():
                if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != d:
                    raise TypeError("dnorm entries must be contiguous fp32 tensors of d elements")
            _require_gpu(*dnorm.values())
            gs = _lib.NormGrads(*[dnorm[k].data_ptr() if dnorm.get(k) is not None else None
                                  for k in ("h_a", "h_b", "r_a", "r_b")])
        rc = lib.kge_build_query_backward_norm(
            MODEL_IDS[model], int(p), int(q), int(r), _ptr(ent), _ptr(rel), _ptr(coeff_p), _ptr(coeff_q), _ptr(coeff_r),
            int(bool(normalize_relation)), ctypes.byref(ns) if ns is not None else None,
            ctypes.byref(gs) if gs is not None else None, dsp, _ptr(hr), B, d, N, R, _ptr(dQ), _ptr(dbias), _ptr(d_ent),
            _ptr(d_rel), _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _stream())
        _lib.check(rc)
        del keep
        return tuple(outs)
    rc = lib.kge_build_query_backward(MODEL_IDS[model], int(p), int(q), int(r), _ptr(ent), _ptr(rel), _ptr(coeff_p),
                                      _ptr(coeff_q), _ptr(coeff_r), int(bool(normalize_relation)), _ptr(hr), B, d, N, R,
                                      _ptr(dQ), _ptr(dbias), _ptr(d_ent), _ptr(d_rel), _ptr(outs[0]), _ptr(outs[1]),
                                      _ptr(outs[2]), _stream())
    _lib.check(rc)
    return tuple(outs)


def scores(Q, bias, E, scale=None, out=None):
    """Materialised [B,N] fp32 scores."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale)
    _check_qe(Q, E, scale, bias)
    B, d = Q.shape
    N = E.shape[0]
    if out is None:
        out = torch.empty((B, N), dtype=torch.float32, device=Q.device)
    _require_gpu(out)
    rc = lib.kge_scores(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, N, _ptr(out),
                        out.stride(0) if B > 0 else N, _stream())
    _lib.check(rc)
    return out


def triple_scores(Q, bias, E, scale, entity):
    """out[b] = Q[b] . E[entity[b]] (* scale) + bias[b]: the score of one given entity per query."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale, entity)
    _check_qe(Q, E, scale, bias)
    if entity.dtype != torch.int64:
        raise TypeError("entity must be int64")
    B, d = Q.shape
    out = torch.empty((B,), dtype=torch.float32, device=Q.device)
    rc = lib.kge_triple_scores(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, E.shape[0],
                               _ptr(entity), _ptr(out), _stream())
    _lib.check(rc)
    return out


def sample_scores(Q, bias, E, scale, entity):
    """out[b, j] = Q[b] . E[entity[b, j]] (* scale) + bias[b] for ``entity`` int64 [B,k]."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale, entity)
    _check_qe(Q, E, scale, bias)
    if entity.dtype != torch.int64 or entity.dim() != 2 or entity.shape[0] != Q.shape[0]:
        raise ValueError("entity must be an int64 tensor of shape [B, k]")
    entity = entity.contiguous()
    B, d = Q.shape
    k = entity.shape[1]
    out = torch.empty((B, k), dtype=torch.float32, device=Q.device)
    rc = lib.kge_sample_scores(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, E.shape[0],
                               _ptr(entity), k, _ptr(out), _stream())
    _lib.check(rc)
    return out


def row_minmax(Q, bias, E, scale=None):
    """(min [B], max [B]) of every query's scores over all entities, without the [B,N] matrix."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale)
    _check_qe(Q, E, scale, bias)
    B, d = Q.shape
    lo = torch.empty((B,), dtype=torch.float32, device=Q.device)
    hi = torch.empty((B,), dtype=torch.float32, device=Q.device)
    rc = lib.kge_row_minmax(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, E.shape[0], _ptr(lo),
                            _ptr(hi), _stream())
    _lib.check(rc)
    return lo, hi


def csr_lookup(hr, keys, num_relations):
    """CSR row of every (h, r) pair of ``hr`` [B,2] in the sorted key array ``keys``; -1 if unknown."""
    lib = _lib.load()
    _require_gpu(hr, keys)
    if hr.dtype != torch.int64 or keys.dtype != torch.int64:
        raise TypeError("hr and keys must be int64")
    B = hr.shape[0]
    out = torch.empty((B,), dtype=torch.int64, device=hr.device)
    rc = lib.kge_csr_lookup(_ptr(hr), B, _ptr(keys) if keys.numel() else None, keys.numel(), int(num_relations),
                            _ptr(out), _stream())
    _lib.check(rc)
    return out


def csr_build(triples, columns, ranges):
    """Sorted, de-duplicated CSR of ``(triples[:, a], triples[:, b]) -> triples[:, v]`` built on the GPU.

    ``triples`` int64 [n,3] on the GPU, ``columns`` = (a, b, v), ``ranges`` = (range_a, range_b, range_v).
    Returns ``keys`` int64 [n_rows] (= a * range_b + b), ``row_ptr`` int64 [n_rows+1], ``col`` int32 [nnz] and
    the number of triples dropped for an out-of-range id.  Reads three integers back (one stream sync)."""
    lib = _lib.load()
    _require_gpu(triples)
    if triples.dtype != torch.int64 or triples.dim() != 2 or triples.shape[1] != 3:
        raise TypeError("triples must be an int64 [n,3] tensor")
    n = triples.shape[0]
    dev = triples.device
    keys = torch.empty((max(n, 1),), dtype=torch.int64, device=dev)
    row_ptr = torch.empty((n + 1,), dtype=torch.int64, device=dev)
    col = torch.empty((max(n, 1),), dtype=torch.int32, device=dev)
    counts = torch.empty((3,), dtype=torch.int64, device=dev)
    ws_bytes = lib.kge_csr_build_workspace_bytes(n)
    if ws_bytes == 0:
        raise _lib.KgeError(-1, lib.kge_last_error().decode("utf-8", "replace"))
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    a, b, v = (int(c) for c in columns)
    ra, rb, rv = (int(r) for r in ranges)
    rc = lib.kge_csr_build(_ptr(triples) if n else None, n, a, b, v, ra, rb, rv, _ptr(keys), _ptr(row_ptr), _ptr(col),
                           _ptr(counts), _ptr(ws), ws_bytes, _stream())
    _lib.check(rc)
    n_rows, nnz, dropped = (int(c) for c in counts.cpu())
    return keys[:n_rows], row_ptr[:n_rows + 1], col[:nnz], dropped


_RANK_OUT = (("n_greater", torch.int32), ("n_equal", torch.int32), ("n_equal_lower", torch.int32),
             ("target_score", torch.float32))


def rank_thresholds(Q, bias, E, scale, target, out):
    """Thresholds (raw target scores) of ANY number of queries in one launch, for ``rank_filtered(..., thr=)``:
    fills ``out`` (dict of [B] tensors as ``rank_filtered`` takes them: the counters initialised, ``target_score``
    written) and returns the fp32 threshold tensor [B]."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale, target)
    _check_qe(Q, E, scale, bias)
    B, d = Q.shape
    if target.dtype != torch.int64:
        raise TypeError("target must be int64")
    for k, dt in _RANK_OUT:
        o = out[k]
        if o.dtype != dt or o.shape != (B,) or o.device != Q.device or not o.is_contiguous():
            raise ValueError(f"out[{k!r}] must be a contiguous {dt} tensor of shape [{B}] on {Q.device}")
    thr = torch.empty((B,), dtype=torch.float32, device=Q.device)
    rc = lib.kge_rank_thresholds(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, E.shape[0],
                                 _ptr(target), _ptr(thr), _ptr(out["n_greater"]), _ptr(out["n_equal"]),
                                 _ptr(out["n_equal_lower"]), _ptr(out["target_score"]), _stream())
    _lib.check(rc)
    return thr


def rank_filtered(Q, bias, E, scale, target, csr_row=None, row_ptr=None, col=None, out=None, thr=None,
                  one_vector_per_row=False):
    """Fused filtered rank. Returns dict of int32 ``n_greater, n_equal, n_equal_lower`` and fp32
    ``target_score`` (all [B]).  ``out``: such a dict of contiguous [B] tensors to write into (slices of an
    evaluation's arrays, say) instead of new ones.  ``thr``: this batch's slice of what ``rank_thresholds`` returned
    for a larger set of queries (``out`` must then be the matching slices of the arrays that call initialised);
    ``one_vector_per_row``: queries that share a filter row are known to hold the same query vector."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale, target, csr_row, row_ptr, col)
    _check_qe(Q, E, scale, bias)
    B, d = Q.shape
    N = E.shape[0]
    dev = Q.device
    if out is None:
        if thr is not None:
            raise ValueError("thr= needs out=: the slices of the arrays that rank_thresholds initialised")
        out = {k: torch.empty((B,), dtype=dt, device=dev) for k, dt in _RANK_OUT}
    else:
        for k, dt in _RANK_OUT:
            o = out[k]
            if o.dtype != dt or o.shape != (B,) or o.device != dev or not o.is_contiguous():
                raise ValueError(f"out[{k!r}] must be a contiguous {dt} tensor of shape [{B}] on {dev}")
    ws_bytes = lib.kge_rank_workspace_bytes(B)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    n_rows = 0 if row_ptr is None else row_ptr.numel() - 1
    if csr_row is not None:
        if csr_row.dtype != torch.int64 or row_ptr.dtype != torch.int64 or col.dtype != torch.int32:
            raise TypeError("csr_row/row_ptr must be int64 and col int32")
    if target.dtype != torch.int64:
        raise TypeError("target must be int64")
    if thr is not None:
        if thr.dtype != torch.float32 or thr.shape != (B,) or thr.device != dev or not thr.is_contiguous():
            raise ValueError(f"thr must be a contiguous float32 tensor of shape [{B}] on {dev}")
        rc = lib.kge_rank_filtered_with_thresholds(
            _ptr(Q), _ptr(E), _table_dtype(E), _ptr(scale), B, d, N, _ptr(target), _ptr(thr), _ptr(csr_row),
            _ptr(row_ptr), _ptr(col), n_rows, int(bool(one_vector_per_row)), _ptr(out["n_greater"]),
            _ptr(out["n_equal"]), _ptr(out["n_equal_lower"]), _ptr(ws), ws_bytes, _stream())
        _lib.check(rc)
        return out
    rc = lib.kge_rank_filtered(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, N, _ptr(target),
                               _ptr(csr_row), _ptr(row_ptr), _ptr(col), n_rows, _ptr(out["n_greater"]),
                               _ptr(out["n_equal"]), _ptr(out["n_equal_lower"]), _ptr(out["target_score"]), _ptr(ws),
                               ws_bytes, _stream())
    _lib.check(rc)
    return out


def topk_prepare(E, scale):
    """The derived form of a table that ``topk`` scans (made once per table and handed to every call as
    ``prepared=``), or None where the storage has none (every storage but per-row int8 with d = 128)."""
    lib = _lib.load()
    _require_gpu(E, scale)
    N, d = E.shape
    nbytes = lib.kge_topk_prepared_bytes(_table_dtype(E), d, N)
    if nbytes == 0:
        return None
    if not E.is_contiguous() or scale is None or not scale.is_contiguous():
        raise ValueError("E and scale must be contiguous")
    buf = torch.empty((nbytes,), dtype=torch.uint8, device=E.device)
    rc = lib.kge_topk_prepare(_ptr(E), _table_dtype(E), _ptr(scale), d, N, _ptr(buf), nbytes, _stream())
    _lib.check(rc)
    return buf


def topk(Q, bias, E, scale, k, sigmoid=False, prepared=None):
    """Fused top-k over all entities: ([B,k] fp32 descending, [B,k] int64).  ``prepared``: what ``topk_prepare``
    returned for this very table (same results, without deriving it again in every call)."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale)
    _check_qe(Q, E, scale, bias)
    B, d = Q.shape
    N = E.shape[0]
    dev = Q.device
    out_s = torch.empty((B, k), dtype=torch.float32, device=dev)
    out_i = torch.empty((B, k), dtype=torch.int64, device=dev)
    if prepared is not None:
        _require_gpu(prepared)
        ws_bytes = lib.kge_topk_prepared_workspace_bytes(B, N, k)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
        rc = lib.kge_topk_prepared(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, N, int(k),
                                   _ptr(out_s), _ptr(out_i), int(bool(sigmoid)), _ptr(prepared), prepared.numel(),
                                   _ptr(ws), ws_bytes, _stream())
    else:
        ws_bytes = lib.kge_topk_workspace_bytes(B, N, k)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
        rc = lib.kge_topk(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, N, int(k), _ptr(out_s),
                          _ptr(out_i), int(bool(sigmoid)), _ptr(ws), ws_bytes, _stream())
    _lib.check(rc)
    return out_s, out_i


def bce_multihot(Q, bias, E, scale, csr_row, row_ptr, col, label_smoothing=0.0):
    """Mean BCE-with-logits of the [B,N] scores against the multi-hot of the CSR rows: [1] fp32 tensor."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, scale, csr_row, row_ptr, col)
    _check_qe(Q, E, scale, bias)
    B, d = Q.shape
    N = E.shape[0]
    loss = torch.empty((1,), dtype=torch.float32, device=Q.device)
    ws_bytes = lib.kge_bce_workspace_bytes()
    ws = torch.empty((ws_bytes // 8,), dtype=torch.float64, device=Q.device)
    n_rows = 0 if row_ptr is None else row_ptr.numel() - 1
    rc = lib.kge_bce_multihot(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), _ptr(scale), B, d, N, _ptr(csr_row),
                              _ptr(row_ptr), _ptr(col), n_rows, float(label_smoothing), _ptr(loss), _ptr(ws),
                              ws_bytes, _stream())
    _lib.check(rc)
    return loss


def bce_multihot_backward(Q, bias, E, csr_row, row_ptr, col, label_smoothing=0.0, grad_out=1.0, want_loss=True):
    """Gradients of ``bce_multihot`` with respect to ``Q`` [B,d], ``bias`` [B] and the fp32 table ``E`` [N,d]:
    ``(loss or None, dQ, dbias, dE)``.  The [B,N] gradient of the scores lives only in the call's workspace."""
    lib = _lib.load()
    _require_gpu(Q, bias, E, csr_row, row_ptr, col)
    _check_qe(Q, E, None, bias)
    if E.dtype != torch.float32:
        raise TypeError("bce_multihot_backward needs an fp32 entity table")
    B, d = Q.shape
    N = E.shape[0]
    loss = torch.empty((1,), dtype=torch.float32, device=Q.device) if want_loss else None
    dQ = torch.empty((B, d), dtype=torch.float32, device=Q.device)
    dbias = torch.empty((B,), dtype=torch.float32, device=Q.device)
    dE = torch.empty((N, d), dtype=torch.float32, device=Q.device)
    ws_bytes = lib.kge_bce_backward_workspace_bytes(B, d, N)
    ws = torch.empty(((ws_bytes + 7) // 8,), dtype=torch.float64, device=Q.device)
    n_rows = 0 if row_ptr is None else row_ptr.numel() - 1
    rc = lib.kge_bce_multihot_backward(_ptr(Q), _ptr(bias), _ptr(E), _table_dtype(E), B, d, N, _ptr(csr_row),
                                       _ptr(row_ptr), _ptr(col), n_rows, float(label_smoothing), float(grad_out),
                                       _ptr(loss), _ptr(dQ), _ptr(dbias), _ptr(dE), _ptr(ws), ws_bytes, _stream())
    _lib.check(rc)
    return loss, dQ, dbias, dE


def profile_begin():
    """Start bracketing every contraction launch with HIP events on its stream."""
    _lib.check(_lib.load().kge_profile_begin())


def profile_end():
    """(total kernel milliseconds, number of launches) since ``profile_begin``; waits for the events."""
    ms = ctypes.c_double(0.0)
    n = ctypes.c_int64(0)
    _lib.check(_lib.load().kge_profile_end(ctypes.byref(ms), ctypes.byref(n)))
    return ms.value, n.value


def profile_kernel():
    """Name (with template arguments) of the main loop most recently timed while profiling was on, as the
    library dispatched it."""
    return _lib.load().kge_profile_kernel().decode("utf-8", "replace")


def probe_mfma(count, reads, seconds=1.0):
    """Measurement aid (``kge_probe_mfma``): the rank main loop's tile statement on random bf16 operands held in
    registers, optionally with its count and with its fragment reads from LDS, for ``seconds``.
    Returns (TFLOP/s of MFMAs issued, milliseconds per launch)."""
    tf, ms = ctypes.c_double(0.0), ctypes.c_double(0.0)
    _lib.check(_lib.load().kge_probe_mfma(int(bool(count)), int(bool(reads)), float(seconds), ctypes.byref(tf),
                                          ctypes.byref(ms), _stream()))
    return tf.value, ms.value


def probe_i8_scan(Q, prepared, N, seconds=1.0):
    """Measurement aid (``kge_probe_i8_scan``): the int8 top-k scan over a prepared table with thresholds of +inf,
    i.e. its hot loop alone.  Returns (tera-operations per second, milliseconds per launch)."""
    assert Q.is_cuda and prepared.is_cuda and Q.dtype == torch.float32 and Q.is_contiguous() and Q.shape[1] == 128
    tf, ms = ctypes.c_double(0.0), ctypes.c_double(0.0)
    _lib.check(_lib.load().kge_probe_i8_scan(Q.data_ptr(), prepared.data_ptr(), Q.shape[0], int(N), float(seconds),
                                             ctypes.byref(tf), ctypes.byref(ms), _stream()))
    return tf.value, ms.value


def probe_walk(Q, E, seconds=1.0):
    """Measurement aid (``kge_probe_walk``): the bf16 d = 128 rank main loop over ``E`` without its count.
    Returns (TFLOP/s, milliseconds per launch)."""
    assert Q.is_cuda and E.is_cuda and Q.dtype == torch.float32 and E.dtype == torch.bfloat16
    assert Q.is_contiguous() and E.is_contiguous() and Q.shape[1] == 128 and E.shape[1] == 128
    tf, ms = ctypes.c_double(0.0), ctypes.c_double(0.0)
    _lib.check(_lib.load().kge_probe_walk(Q.data_ptr(), E.data_ptr(), Q.shape[0], E.shape[0], float(seconds),
                                          ctypes.byref(tf), ctypes.byref(ms), _stream()))
    return tf.value, ms.value
