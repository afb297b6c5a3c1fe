"""Full-size checks (the benchmark's own shapes) through size-independent properties.

At 2.5M / 10M entities the CPU oracle cannot score a whole batch, so the fused kernels are checked
against the library's materialised scores of a few sampled queries (bit-exact), against themselves
under a different batch composition (bit-exact), and through counting identities.
"""
import numpy as np
import pytest
import torch

from oracle import kge_oracle as ko

pytestmark = pytest.mark.gpu


def test_c2_complex_filtered_mrr_eval_at_full_size():
    """The second benchmark configuration as it is specified: ComplEx, 14,541 entities, d = 200 fp32, 272k Zipf triples, 20k eval queries in
    batches of 1024 (the last holds 544) through the Evaluator (dicee/evaluation/evaluator.py:473-510).  Every rank
    lies inside the fp64 oracle's tolerance interval and equals the oracle's rank wherever that interval is one
    point; the counters of sampled batches are bit-exact against the library's own materialised scores."""
    from types import SimpleNamespace
    from dicee_amd import synthetic
    from dicee_amd.evaluator import Evaluator
    cfg = synthetic.make_config("c2")
    assert (cfg.N, cfg.R, cfg.d, cfg.B, len(cfg.queries), len(cfg.triples)) == (14541, 237, 200, 1024, 20000, 272000)
    model = synthetic.make_model(cfg, torch.device("cuda:0"))
    ev = Evaluator(SimpleNamespace(batch_size=cfg.B, eval_model="test", scoring_technique="KvsAll",
                                   full_storage_path=None))
    ev.set_filter(cfg.csr)
    res = ev.evaluate_lp_k_vs_all(model, cfg.queries)
    ranks = ev.last_ranks
    assert ranks.shape == (20000,)
    exact = inside = 0
    for i in range(0, len(cfg.queries), cfg.B):
        q = cfg.queries[i:i + cfg.B]
        S = ko.k_vs_all_scores("ComplEx", cfg.E, cfg.Rel, q[:, :2])          # fp64 [<=1024, 14541]
        rms = np.sqrt((S ** 2).mean(axis=1))
        for j, (h, r, t) in enumerate(q):
            filt = cfg.csr.tails(int(h), int(r))
            tol = 1e-5 * max(abs(S[j, t]), rms[j])
            lo, hi = ko.rank_interval_with_tolerance(S[j], int(t), filt, tol)
            inside += lo <= ranks[i + j] <= hi
            exact += lo == hi
    assert inside == len(cfg.queries)
    assert exact > 0.8 * len(cfg.queries)            # the interval is one point (the rank is pinned exactly) for most
    want = ko.metrics_from_ranks(ranks)
    for key in ("H@1", "H@3", "H@10", "MRR"):
        assert res[key] == pytest.approx(want[key], rel=1e-12)
    # counters bit-exact against the library's own scores: first batch, last (544-query) batch
    cfg.csr.to("cuda")
    for i in (0, 19 * cfg.B):
        q = torch.from_numpy(cfg.queries[i:i + cfg.B].copy()).cuda()
        x, t = q[:, :2].contiguous(), q[:, 2].contiguous()
        c = model.rank_filtered(x, t, cfg.csr)
        S = model(x).cpu().numpy()
        tt = t.cpu().numpy()
        for j in range(len(tt)):
            filt = cfg.csr.tails(int(x[j, 0]), int(x[j, 1]))
            g, e, el = ko.filtered_rank_counts(S[j], int(tt[j]), filt)
            assert (g, e, el) == (int(c["n_greater"][j]), int(c["n_equal"][j]), int(c["n_equal_lower"][j]))


@pytest.fixture(scope="module")
def c4():
    from dicee_amd import synthetic
    cfg = synthetic.make_config("c4", with_tables=False)
    model = synthetic.make_model(cfg, torch.device("cuda:0"), tables_on_device=True)
    cfg.csr.to("cuda")
    return cfg, model


def test_c4_fused_rank_matches_materialised_scores_and_is_batch_invariant(c4):
    cfg, model = c4
    q = torch.from_numpy(cfg.queries[:4096].copy()).cuda()
    x, t = q[:, :2].contiguous(), q[:, 2].contiguous()
    full = model.rank_filtered(x, t, cfg.csr)
    plain = model.rank_filtered(x, t, None)
    # sample: the queries with the longest filter rows, some ordinary ones, and the last of the batch
    rows = cfg.csr.rows_for_numpy(cfg.queries[:4096, :2])
    lens = np.diff(cfg.csr.row_ptr_np)[rows]
    pick = np.unique(np.concatenate([np.argsort(-lens)[:3], np.arange(0, 4096, 1000), [4095]]))
    xs, ts = x[pick].contiguous(), t[pick].contiguous()
    small = model.rank_filtered(xs, ts, cfg.csr)
    for key in ("n_greater", "n_equal", "n_equal_lower", "target_score"):
        assert torch.equal(small[key], full[key][pick]), key          # same bits in a batch of 8 or 4096
    S = model(xs).cpu().numpy()                                        # [len(pick), 2.5M] materialised
    assert lens[pick].max() >= 10000
    for j, b in enumerate(pick):
        h, r, tt = (int(v) for v in cfg.queries[b])
        filt = cfg.csr.tails(h, r)
        g, e, el = ko.filtered_rank_counts(S[j], tt, filt)
        assert (g, e, el) == (int(full["n_greater"][b]), int(full["n_equal"][b]), int(full["n_equal_lower"][b]))
        g0, e0, el0 = ko.filtered_rank_counts(S[j], tt, None)
        assert (g0, e0, el0) == (int(plain["n_greater"][b]), int(plain["n_equal"][b]),
                                 int(plain["n_equal_lower"][b]))
        assert float(full["target_score"][b]) == S[j, tt]
    # counting identities over the whole batch
    ng, ng0 = full["n_greater"].cpu().numpy(), plain["n_greater"].cpu().numpy()
    assert np.all(ng >= 0) and np.all(ng <= ng0) and np.all(ng0 < cfg.N)
    assert np.all(ng0 - ng <= lens)                                    # at most the filter row is removed
    assert np.all(plain["n_equal"].cpu().numpy() >= full["n_equal"].cpu().numpy())


def test_c4_topk_matches_materialised_scores(c4):
    cfg, model = c4
    q = torch.from_numpy(cfg.queries[4096:4096 + 600, :2].copy()).cuda()
    vals, idx = model.topk(q, cfg.k)
    sub = q[::100].contiguous()
    S = model(sub).cpu().numpy()
    wv, wi = ko.topk(S, cfg.k)
    np.testing.assert_array_equal(idx[::100].cpu().numpy(), wi)
    np.testing.assert_array_equal(vals[::100].cpu().numpy(), wv)
    v2, i2 = model.topk(sub, cfg.k)                                    # batch-size invariance
    assert torch.equal(i2, idx[::100]) and torch.equal(v2, vals[::100])
    assert bool((vals[:, :-1] >= vals[:, 1:]).all())                   # sorted descending


def test_c4_vocabularies_built_on_the_gpu_and_head_direction(c4):
    """10M triples -> (h, r) and (r, t) vocabularies on the GPU; the first against the numpy builder, the second
    used to rank true heads, checked against materialised head-direction scores of sampled queries."""
    from dicee_amd.csr import FilterCSR
    cfg, model = c4
    trip = torch.from_numpy(cfg.triples).cuda()
    er = FilterCSR.from_triples_gpu(trip, cfg.N, cfg.R, kind="er")
    host = FilterCSR.from_triples(cfg.triples, cfg.R)                  # no per-row cap, unlike cfg.csr
    assert torch.equal(er.keys.cpu(), torch.from_numpy(host.keys_np))
    assert torch.equal(er.row_ptr.cpu(), torch.from_numpy(host.row_ptr_np))
    assert torch.equal(er.col.cpu(), torch.from_numpy(host.col_np))
    re = FilterCSR.from_triples_gpu(trip, cfg.N, cfg.R, kind="re")
    assert re.nnz == er.nnz                                            # both hold every distinct triple once
    q = torch.from_numpy(cfg.queries[:2048].copy()).cuda()
    rt, h = q[:, 1:].contiguous(), q[:, 0].contiguous()
    full = model.rank_filtered(rt, h, re, heads=True)
    lens = np.diff(re.row_ptr_np)[re.rows_for_numpy(cfg.queries[:2048, 1:])]
    pick = np.unique(np.concatenate([np.argsort(-lens)[:2], [0, 777, 2047]]))
    S = model.forward_all_heads(rt[pick].contiguous()).cpu().numpy()
    for j, b in enumerate(pick):
        hh, r, t = (int(v) for v in cfg.queries[b])
        heads = re.col_np[re.row_ptr_np[re.rows_for_numpy(np.array([[r, t]]))[0]]:][:lens[b]]
        g, e, el = ko.filtered_rank_counts(S[j], hh, heads)
        assert (g, e, el) == (int(full["n_greater"][b]), int(full["n_equal"][b]), int(full["n_equal_lower"][b]))
        assert float(full["target_score"][b]) == S[j, hh]
    # one triple, both directions: the head-direction score of (r, t) at h equals the tail-direction score of (h, r) at t
    both = model.forward_triples(q[:2048])
    err = (full["target_score"] - both).abs()                          # different bf16 roundings of the two query vectors
    assert float(err.max()) <= 2e-2 * float(both.pow(2).mean().sqrt())


def test_c5_int8_topk_matches_materialised_scores():
    from dicee_amd import synthetic
    cfg = synthetic.make_config("c5", with_tables=False)
    model = synthetic.make_model(cfg, torch.device("cuda:0"), tables_on_device=True)
    assert model.table()[0].dtype == torch.int8 and model.table()[0].shape == (10_000_000, 128)
    q = torch.from_numpy(cfg.queries[:512, :2].copy()).cuda()
    vals, idx = model.topk(q, cfg.k)
    sub = q[::128].contiguous()
    S = model(sub).cpu().numpy()
    wv, wi = ko.topk(S, cfg.k)
    np.testing.assert_array_equal(idx[::128].cpu().numpy(), wi)
    np.testing.assert_array_equal(vals[::128].cpu().numpy(), wv)
    # scores follow fp32 math on the dequantised table within the int8 bar
    E, scale = model.table()
    rows = wi[0]
    deq = (E[torch.from_numpy(rows).cuda()].float() * scale[torch.from_numpy(rows).cuda()][:, None]).cpu().numpy()
    Q, _ = model.query(sub[:1])
    ref = deq.astype(np.float64) @ Q[0].cpu().numpy().astype(np.float64)
    np.testing.assert_allclose(wv[0], ref, rtol=2e-2)
    del model
    torch.cuda.empty_cache()


def test_c3_bce_step_and_its_backward_at_full_size():
    """C3 (N=40,943, d=256, fp32, batch 2048): the fused loss against the library's own materialised scores, and
    the gradients through identities that hold for any size: dE^T 1 = Q^T dbias, <dQ, Q> = <dE, E> = <g, S - bias>,
    linearity in the upstream gradient, and a sampled block of dQ / dE against fp64 products of the dense gradient."""
    from dicee_amd import synthetic, ops
    cfg = synthetic.make_config("c3")
    model = synthetic.make_model(cfg, torch.device("cuda:0"))
    cfg.csr.to("cuda")
    x = torch.from_numpy(cfg.queries[:cfg.B, :2].copy()).cuda()
    eps = 0.1
    loss, dQ, dbias, dE = model.kvsall_bce_backward(x, cfg.csr, label_smoothing=eps)
    assert loss.item() == pytest.approx(model.kvsall_bce_loss(x, cfg.csr, label_smoothing=eps).item(), rel=1e-6)
    Q, bias = model.query(x)
    E, _ = model.table()
    S = ops.scores(Q, bias, E).double()                                 # [2048, 40943]
    rows = cfg.csr.rows_for(x)
    y = torch.full_like(S, 1.0 / cfg.N)
    rp, col = cfg.csr.row_ptr.cpu().numpy(), cfg.csr.col.cpu().numpy()
    for b, r in enumerate(rows.cpu().numpy()):
        if r >= 0:
            y[b, col[rp[r]:rp[r + 1]].astype(np.int64)] += 1.0 - eps
    want_loss = torch.nn.functional.binary_cross_entropy_with_logits(S, y).item()
    assert loss.item() == pytest.approx(want_loss, rel=1e-5)
    g = (torch.sigmoid(S) - y) / (cfg.B * cfg.N)
    del y
    Qd, Ed = Q.double(), E.double()
    # fp32 sums of 40,943 (dQ, dbias) or 2048 (dE) products that largely cancel: bound each element by the sum of
    # the magnitudes of its terms (2e-6 of it: a few units of fp32 rounding per term at most)
    ga = g.abs()
    for got, want, mag, name in ((dQ, g @ Ed, ga @ Ed.abs(), "dQ"), (dE, g.T @ Qd, ga.T @ Qd.abs(), "dE"),
                                 (dbias, g.sum(1), ga.sum(1), "dbias")):
        worst = ((got.double() - want).abs() / mag).max().item()
        assert worst <= 2e-6, (name, worst)
    del ga
    # identities on the fp32 results themselves
    lhs, rhs = dE.double().sum(0), dbias.double() @ Qd
    assert (lhs - rhs).abs().max().item() <= 1e-5 * rhs.abs().max().item() + 1e-12
    a, b = (dQ.double() * Qd).sum().item(), (dE.double() * Ed).sum().item()
    assert a == pytest.approx(b, rel=1e-5)
    _, dQ2, dbias2, dE2 = model.kvsall_bce_backward(x, cfg.csr, label_smoothing=eps, grad_out=2.0)
    for one, two in ((dQ, dQ2), (dE, dE2)):
        assert torch.equal(one * 2.0, two)                             # a power of two scales every product exactly
    # the row sums are gathered with floating-point atomics: same value up to the order of the additions
    assert (dbias2 - 2.0 * dbias).abs().max().item() <= 2e-6 * 2.0 * g.abs().sum(1).max().item()
