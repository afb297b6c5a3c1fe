"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

from oracle import kge_oracle as ko

RTOL = {"fp32": 1e-5, "bf16": 2e-2, "int8": 2e-2}


def score_close(got, ref, rtol):
    """|got - ref| <= rtol * max(|ref|, row RMS of ref): scores are sums of signed products, so a
    purely relative bound is meaningless near zero."""
    ref = np.asarray(ref, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    if ref.ndim == 1:
        rms = np.sqrt((ref ** 2).mean()) if ref.size else 0.0
        bound = rtol * np.maximum(np.abs(ref), rms)
    else:
        rms = np.sqrt((ref ** 2).mean(axis=1, keepdims=True))
        bound = rtol * np.maximum(np.abs(ref), rms)
    err = np.abs(got - ref)
    worst = float((err / np.maximum(bound, 1e-300)).max()) if err.size else 0.0
    return bool((err <= bound).all()), worst


def random_tables(rng, N, R, d, std=0.1):
    E = (rng.standard_normal((N, d)) * std).astype(np.float32)
    Rel = (rng.standard_normal((R, d)) * std).astype(np.float32)
    return E, Rel


def random_hr(rng, N, R, B):
    return np.stack([rng.integers(0, N, B), rng.integers(0, R, B)], axis=1).astype(np.int64)


def stored_tables(E, Rel, storage):
    """(E as the kernels see it [torch cpu tensor], scale or None, Rel tensor, E / Rel as the fp32 values
    the oracle must use)."""
    if storage == "fp32":
        return torch.from_numpy(E), None, torch.from_numpy(Rel), E, Rel
    if storage == "bf16":
        Eb, Rb = ko.bf16_round(E), ko.bf16_round(Rel)
        return (torch.from_numpy(Eb).to(torch.bfloat16), None, torch.from_numpy(Rb).to(torch.bfloat16), Eb, Rb)
    if storage == "int8":
        q, s = ko.quantize_int8_rows(E)
        return torch.from_numpy(q), torch.from_numpy(s), torch.from_numpy(Rel), ko.dequantize_int8_rows(q, s), Rel
    raise ValueError(storage)


def dev(t, device="cuda"):
    return None if t is None else t.to(device).contiguous()


def random_csr(rng, hr, targets, N, R, max_len=6, include_target=0.5, hub_rows=()):
    """er_vocab-like dict for the (h, r) pairs of ``hr``; ``hub_rows``: list of (index into hr, length)."""
    er = {}
    for j, (h, r) in enumerate(hr):
        key = (int(h), int(r))
        lst = er.setdefault(key, [])
        lst.extend(int(v) for v in rng.integers(0, N, rng.integers(0, max_len + 1)))
        if rng.random() < include_target:
            lst.append(int(targets[j]))
    for j, length in hub_rows:
        key = (int(hr[j, 0]), int(hr[j, 1]))
        er[key].extend(int(v) for v in rng.choice(N, size=length, replace=False))
    return er
