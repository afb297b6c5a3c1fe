"""Seeded synthetic knowledge graphs and embedding tables for the five benchmark configurations.

There is no network for datasets or checkpoints, so every workload is generated: entity / relation
tables drawn N(0, std), triples with Zipf-distributed slots (probability proportional to
rank^-a over a FINITE support, mapped through a random permutation of the ids).
"""
from types import SimpleNamespace

import numpy as np

from .csr import FilterCSR

CONFIGS = {
    # DistMult KvsAll scoring + filtered rank on a toy KG
    "c1": dict(model="DistMult", N=135, R=46, d=32, n_triples=5216, B=512, n_queries=512, seed=0, std=0.1,
               storage="fp32", zipf_h=None, zipf_t=None, zipf_r=1.1, k=10),
    # ComplEx KvsAll + filtered MRR
    "c2": dict(model="ComplEx", N=14541, R=237, d=200, n_triples=272000, B=1024, n_queries=20000, seed=1, std=0.1,
               storage="fp32", zipf_h=1.05, zipf_t=1.05, zipf_r=1.2, k=10),
    # Keci(0,1) KvsAll forward + BCE over the multi-hot target
    "c3": dict(model="Keci", p=0, q=1, N=40943, R=18, d=256, n_triples=87000, B=2048, n_queries=2048, seed=2,
               std=0.1, storage="fp32", zipf_h=1.3, zipf_t=1.3, zipf_r=None, k=10, max_per_row=400),
    # QMult filtered rank + top-10 at scale, bf16 storage
    "c4": dict(model="QMult", N=2500000, R=37, d=128, n_triples=10000000, B=4096, n_queries=50000, seed=3, std=0.05,
               storage="bf16", zipf_h=1.1, zipf_t=1.1, zipf_r=1.2, k=10, max_per_row=50000),
    # DistMult top-100 over an int8 table, no filter
    "c5": dict(model="DistMult", N=10000000, R=1000, d=128, n_triples=0, B=8192, n_queries=8192, seed=4, std=0.1,
               storage="int8", zipf_h=None, zipf_t=None, zipf_r=None, k=100),
}


def zipf_probs(n, a):
    p = np.arange(1, n + 1, dtype=np.float64) ** (-float(a))
    return p / p.sum()


def zipf_sample(rng, n, a, size):
    """``size`` ids in [0,n): uniform if ``a`` is None, else Zipf(a) over a random permutation."""
    if a is None:
        return rng.integers(0, n, size=size, dtype=np.int64)
    cdf = np.cumsum(zipf_probs(n, a))
    cdf[-1] = 1.0
    ranks = np.searchsorted(cdf, rng.random(size), side="right").astype(np.int64)
    return rng.permutation(n).astype(np.int64)[np.minimum(ranks, n - 1)]


def make_config(name, scale=1.0, with_tables=True):
    """Workload ``name`` (``c1``..``c5``), optionally shrunk: ``scale`` < 1 multiplies the entity,
    triple and query counts (distributions and dims unchanged).  Returns a namespace with numpy
    ``E`` [N,d], ``Rel`` [R,d] (fp32; omitted if ``with_tables`` is False), ``triples`` [n,3],
    ``queries`` [n_queries,3] (h, r, true tail), ``csr`` (FilterCSR over all triples) and the
    configuration fields."""
    c = dict(CONFIGS[name])
    if scale != 1.0:
        c["N"] = max(64, int(c["N"] * scale))
        c["n_triples"] = int(c["n_triples"] * scale)
        c["n_queries"] = max(1, int(c["n_queries"] * scale))
    rng = np.random.default_rng(c["seed"])
    N, R, d = c["N"], c["R"], c["d"]
    out = SimpleNamespace(name=name, **c)
    if with_tables:
        out.E = (rng.standard_normal((N, d), dtype=np.float32) * np.float32(c["std"]))
        out.Rel = (rng.standard_normal((R, d), dtype=np.float32) * np.float32(c["std"]))
    n = c["n_triples"]
    if n > 0:
        h = zipf_sample(rng, N, c["zipf_h"], n)
        r = zipf_sample(rng, R, c["zipf_r"], n)
        t = zipf_sample(rng, N, c["zipf_t"], n)
        triples = np.stack([h, r, t], axis=1)
        out.csr = FilterCSR.from_triples(triples, R, max_per_row=c.get("max_per_row"))
        if name == "c3":
            # KvsAll training rows: the first B unique (h, r) pairs in key order, no targets
            keys = out.csr.keys_np[:c["n_queries"]]
            out.queries = np.stack([keys // R, keys % R, np.zeros_like(keys)], axis=1)
        elif name == "c1":
            out.queries = triples[:c["n_queries"]].copy()
        else:
            pick = rng.choice(n, size=c["n_queries"], replace=n < c["n_queries"])
            out.queries = triples[pick].copy()
        out.triples = triples
    else:
        out.csr = None
        out.triples = np.empty((0, 3), dtype=np.int64)
        out.queries = np.stack([rng.integers(0, N, c["n_queries"]), rng.integers(0, R, c["n_queries"]),
                                rng.integers(0, N, c["n_queries"])], axis=1).astype(np.int64)
    return out


def make_model(cfg, device, tables_on_device=False):
    """A ``dicee_amd`` model for ``cfg`` on ``device`` with the configuration's storage.  With
    ``tables_on_device`` the tables are drawn on the GPU (seeded torch generator) instead of being
    copied from ``cfg.E`` / ``cfg.Rel``: used at full size where the host copy would dominate."""
    import torch
    from .models import MODEL_REGISTRY
    args = {"model": cfg.model, "embedding_dim": cfg.d, "num_entities": cfg.N, "num_relations": cfg.R,
            "p": getattr(cfg, "p", 0), "q": getattr(cfg, "q", 0)}
    name = "CKeci" if cfg.model == "Keci" else cfg.model        # benchmark Keci with unit coefficients
    with torch.device("meta"):
        model = MODEL_REGISTRY[name](args)
    model = model.to_empty(device=device)
    with torch.no_grad():
        if tables_on_device:
            g = torch.Generator(device=device)
            g.manual_seed(cfg.seed)
            model.entity_embeddings.weight.normal_(0.0, cfg.std, generator=g)
            model.relation_embeddings.weight.normal_(0.0, cfg.std, generator=g)
        else:
            model.entity_embeddings.weight.copy_(torch.from_numpy(cfg.E))
            model.relation_embeddings.weight.copy_(torch.from_numpy(cfg.Rel))
        if hasattr(model, "p_coefficients"):
            model.p_coefficients.weight.fill_(1.0)
        if hasattr(model, "q_coefficients"):
            model.q_coefficients.weight.fill_(1.0)
    for p_ in model.parameters():
        p_.requires_grad_(False)
    model.eval()
    model.set_entity_storage(cfg.storage)
    return model
