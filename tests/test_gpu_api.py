"""The Python call surface (models, Evaluator, KGE) on the GPU against the oracle, including the
consistency checks the reference's own tests make: two rank loops agree exactly
(tests/test_link_prediction_evaluation.py:98-107), ``predict`` is deterministic
(tests/test_predict_kge.py:68-73), ``predict_topk`` equals ``sigmoid(predict)`` at the same entity
within 1e-6 (:85-95) and is identical for batch sizes 1, 2, 4, 8 (:107-119)."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from helpers import score_close
from oracle import kge_oracle as ko
from oracle import torch_cpu_path as tcp

pytestmark = pytest.mark.gpu


def _toy(model_name, d, N=135, R=46, n=2000, seed=0, **extra):
    from dicee_amd import models
    rng = np.random.default_rng(seed)
    args = {"model": model_name, "embedding_dim": d, "num_entities": N, "num_relations": R, **extra}
    torch.manual_seed(seed)
    m = models.MODEL_REGISTRY[model_name](args)
    with torch.no_grad():
        m.entity_embeddings.weight.normal_(0, 0.1)
        m.relation_embeddings.weight.normal_(0, 0.1)
        if hasattr(m, "p_coefficients"):
            m.p_coefficients.weight.normal_(1.0, 0.3)
        if hasattr(m, "q_coefficients"):
            m.q_coefficients.weight.normal_(1.0, 0.3)
        if hasattr(m, "r_coefficients"):
            m.r_coefficients.weight.normal_(1.0, 0.3)
    triples = np.stack([rng.integers(0, N, n), rng.integers(0, R, n), rng.integers(0, N, n)], axis=1)
    return m, triples


def _oracle_kw(m):
    kw = {}
    if m.name in ("Keci", "CKeci"):
        kw = {"p": m.p, "q": m.q}
        if m.p:
            kw["coeff_p"] = m.p_coefficients.weight.detach().cpu().numpy().reshape(-1)
        if m.q:
            kw["coeff_q"] = m.q_coefficients.weight.detach().cpu().numpy().reshape(-1)
    if m.name == "DeCaL":
        kw = {"p": m.p, "q": m.q, "r": m.r}
        for n, key, attr in ((m.p, "coeff_p", "p_coefficients"), (m.q, "coeff_q", "q_coefficients"),
                             (m.r, "coeff_r", "r_coefficients")):
            if n:
                kw[key] = getattr(m, attr).weight.detach().cpu().numpy().reshape(-1)
    return kw


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("ComplEx", 32, {}), ("QMult", 32, {}),
                                          ("OMult", 32, {}),
                                          ("Keci", 30, {"p": 2, "q": 2}), ("CKeci", 32, {"p": 0, "q": 1}),
                                          ("DeCaL", 32, {"p": 2, "q": 2, "r": 3}), ("DeCaL", 30, {"p": 1, "q": 1, "r": 3})])
def test_forward_k_vs_all_is_a_drop_in(name, d, extra):
    m, triples = _toy(name, d, **extra)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    kw = _oracle_kw(m)
    m = m.to("cuda").eval()
    x = torch.from_numpy(triples[:200, :2].copy()).cuda()
    with torch.no_grad():
        S = m(x)                                                  # BaseKGE.forward shape dispatch
    assert S.shape == (200, 135) and S.dtype == torch.float32 and S.is_cuda
    ref = ko.k_vs_all_scores("Keci" if name == "CKeci" else name, E, Rel, triples[:200, :2], **kw)
    ok, worst = score_close(S.cpu().numpy(), ref, 1e-5)
    assert ok, worst
    S[0, :5] = -np.inf                                            # callers mutate the result in place
    # k_vs_all_score on gathered rows
    S2 = m.k_vs_all_score(m.entity_embeddings(x[:, 0]), m.relation_embeddings(x[:, 1]), m.entity_embeddings.weight)
    ok, worst = score_close(S2.cpu().numpy(), ref, 1e-5)
    assert ok, worst


@pytest.mark.parametrize("d,batch_size", [(50, 3), (25, 7), (50, 64)])
def test_evaluation_in_batches_whose_query_rows_are_not_16_byte_aligned(d, batch_size):
    """The evaluation loop builds the query vectors of many batches at once and hands row slices to the library,
    which wants 16-byte aligned operands: with d % 4 != 0 and an odd batch size the slices of every batch after the
    first start off alignment and are copied first.  Ranks equal those of one call over all queries."""
    from dicee_amd.evaluator import rank_in_batches, ranks_from_counts
    from dicee_amd.csr import FilterCSR
    m, triples = _toy("DistMult", d, n=400, seed=11)
    m = m.to("cuda").eval()
    csr = FilterCSR.from_triples(triples, 46)
    csr.to("cuda")
    x = torch.from_numpy(triples[:100, :2].copy()).cuda()
    t = torch.from_numpy(triples[:100, 2].copy()).cuda()
    got = rank_in_batches(m, x, t, csr, batch_size, call_queries=0)      # one call per batch
    c = m.rank_filtered(x, t, csr)
    want = ranks_from_counts(c["n_greater"], c["n_equal"], c["n_equal_lower"])
    assert torch.equal(got, want)
    # whole batches merged into calls of at least ten queries (still off alignment), and into one call (the default
    # merges up to 8192 queries): the same ranks
    assert torch.equal(rank_in_batches(m, x, t, csr, batch_size, call_queries=10), want)
    assert torch.equal(rank_in_batches(m, x, t, csr, batch_size), want)
    S = ko.k_vs_all_scores("DistMult", m.entity_embeddings.weight.detach().cpu().numpy(),
                           m.relation_embeddings.weight.detach().cpu().numpy(), triples[:100, :2])
    for j, (h, r, tt) in enumerate(triples[:100]):
        lo, hi = ko.rank_interval_with_tolerance(S[j], int(tt), csr.tails(int(h), int(r)), 1e-5 * np.sqrt((S[j] ** 2).mean()))
        assert lo <= int(got[j]) <= hi


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("ComplEx", 64, {}), ("QMult", 64, {}),
                                          ("Keci", 48, {"p": 1, "q": 1})])
@pytest.mark.parametrize("batch_size", [64, 1000])
def test_evaluator_matches_the_reference_loop(name, d, extra, batch_size):
    from dicee_amd import Evaluator
    m, triples = _toy(name, d, n=1500, seed=3, **extra)
    E = m.entity_embeddings.weight.detach().clone()
    Rel = m.relation_embeddings.weight.detach().clone()
    kw = _oracle_kw(m)
    er = {}
    for h, r, t in triples:
        er.setdefault((int(h), int(r)), []).append(int(t))
    ds = SimpleNamespace(num_entities=135, num_relations=46, er_vocab=er, train_set=triples,
                         valid_set=triples[:300], test_set=triples[300:700])
    ev = Evaluator(SimpleNamespace(batch_size=batch_size, eval_model="train_val_test", scoring_technique="KvsAll",
                                   full_storage_path=None))
    m = m.to("cuda")
    report = ev.eval(ds, m, "EntityPrediction", during_training=True)
    assert set(report) == {"Train", "Val", "Test"}
    assert set(report["Test"]) == {"H@1", "H@3", "H@10", "MRR"}
    # the reference's op sequence on torch CPU (mask loop + unstable sort)
    tkw = {k: (torch.tensor(v) if k.startswith("coeff") else v) for k, v in kw.items()}
    ref_ranks = tcp.evaluate_entity_prediction("Keci" if name == "CKeci" else name, E, Rel, triples[300:700], er,
                                               batch_size, **tkw)
    got = ev.last_ranks
    # every rank inside the fp64 oracle's tolerance interval; identical to the CPU loop except at near-ties
    S = ko.k_vs_all_scores(name, E.numpy(), Rel.numpy(), triples[300:700, :2], **kw)
    for j, (h, r, t) in enumerate(triples[300:700]):
        tol = 1e-5 * np.sqrt((S[j] ** 2).mean())
        lo, hi = ko.rank_interval_with_tolerance(S[j], int(t), er[(int(h), int(r))], tol)
        assert lo <= got[j] <= hi
        if lo == hi:
            assert got[j] == ref_ranks[j]
    agree = np.mean(np.asarray(ref_ranks) == got)
    assert agree >= 0.99
    want = ko.metrics_from_ranks(got)
    assert report["Test"]["MRR"] == pytest.approx(want["MRR"]) and report["Test"]["H@10"] == want["H@10"]
    # the counters-based evaluator and an evaluation on materialised scores agree exactly
    x = torch.from_numpy(triples[300:700, :2].copy()).cuda()
    with torch.no_grad():
        Sg = m(x).cpu().numpy() - m.query(x)[1].cpu().numpy()[:, None]
    if name != "Keci":
        own = ko.filtered_ranks(Sg, triples[300:700, 2], [er[(int(h), int(r))] for h, r, _ in triples[300:700]])
        np.testing.assert_array_equal(own, got)


@pytest.mark.parametrize("storage", ["fp32", "bf16", "int8"])
def test_evaluator_batches_on_alternating_streams_give_the_same_ranks(storage):
    """The batches of an evaluation alternate over two streams by default.  Whatever the number of streams, the ranks
    are those of the one-stream evaluation; with quantised storage the table's snapshot is taken lazily by the first
    batch, before the streams fork.  (Batches of 512 against 3000 entities: above the size below which the evaluator
    keeps to one stream.)"""
    from dicee_amd import Evaluator
    m, triples = _toy("DistMult", 64, N=3000, R=11, n=6000, seed=11)
    er = {}
    for h, r, t in triples:
        er.setdefault((int(h), int(r)), []).append(int(t))
    ranks = {}
    for streams in (1, 2, 3):
        model = m.to("cuda").set_entity_storage(storage)           # (a fresh snapshot for every run)
        ev = Evaluator(SimpleNamespace(batch_size=512, eval_model="test", scoring_technique="KvsAll",
                                       full_storage_path=None), streams=streams)
        ev.set_filter(er, num_relations=11)
        ev.evaluate_lp_k_vs_all(model, triples, form_of_labelling="EntityPrediction")
        ranks[streams] = ev.last_ranks.copy()
    np.testing.assert_array_equal(ranks[1], ranks[2])
    np.testing.assert_array_equal(ranks[1], ranks[3])
    assert len(ranks[1]) == len(triples) and ranks[1].min() >= 1
    # more batches than one group holds (64): the groups' vectors and rows are made, used and released in turn; the
    # ranks do not depend on how the triples are cut into batches and groups
    rng = np.random.default_rng(3)
    many = np.stack([rng.integers(0, 3000, 40000), rng.integers(0, 11, 40000), rng.integers(0, 3000, 40000)], axis=1)
    by_cut = {}
    for bs, streams in ((512, 2), (512, 1), (4096, 2)):
        ev = Evaluator(SimpleNamespace(batch_size=bs, eval_model="test", scoring_technique="KvsAll",
                                       full_storage_path=None), streams=streams)
        ev.set_filter(er, num_relations=11)
        ev.evaluate_lp_k_vs_all(model, many, form_of_labelling="EntityPrediction")
        by_cut[(bs, streams)] = ev.last_ranks.copy()
    np.testing.assert_array_equal(by_cut[(512, 2)], by_cut[(512, 1)])
    np.testing.assert_array_equal(by_cut[(512, 2)], by_cut[(4096, 2)])
    # called on a stream of the caller's: the evaluation forks from it, joins it and leaves it current
    mine = torch.cuda.Stream()
    with torch.cuda.stream(mine):
        ev = Evaluator(SimpleNamespace(batch_size=512, eval_model="test", scoring_technique="KvsAll",
                                       full_storage_path=None), streams=2)
        ev.set_filter(er, num_relations=11)
        ev.evaluate_lp_k_vs_all(model, triples, form_of_labelling="EntityPrediction")
        assert torch.cuda.current_stream() == mine
    np.testing.assert_array_equal(ev.last_ranks, ranks[1])
    assert torch.cuda.current_stream() == torch.cuda.default_stream()
    # the head-and-tail evaluation: two rank calls per batch, on alternating streams as well
    from dicee_amd import FilterCSR
    from dicee_amd.link_prediction import evaluate_lp
    model = m.to("cuda").set_entity_storage(storage)
    dev_trip = torch.from_numpy(triples.astype(np.int64)).cuda()
    er_csr = FilterCSR.from_triples_gpu(dev_trip, 3000, 11, kind="er")
    re_csr = FilterCSR.from_triples_gpu(dev_trip, 3000, 11, kind="re")
    both = {s: evaluate_lp(model, triples, 3000, er_csr, re_csr, info=None, batch_size=512, return_ranks=True,
                           streams=s) for s in (1, 2, 3)}
    for s in (2, 3):
        assert both[s][0] == both[1][0]
        np.testing.assert_array_equal(both[s][1][0], both[1][1][0])
        np.testing.assert_array_equal(both[s][1][1], both[1][1][1])


def test_rank_counters_written_into_the_callers_arrays():
    """``out=``: a batch writes its counters into slices of the evaluation's arrays (what the evaluator's loop does);
    the same numbers as the call that allocates, and arrays of another type, length or layout are refused."""
    from dicee_amd import FilterCSR
    m, triples = _toy("ComplEx", 64, N=900, R=7, n=700, seed=5)
    m = m.to("cuda").eval()
    trip = torch.from_numpy(triples.astype(np.int64)).cuda()
    csr = FilterCSR.from_triples_gpu(trip, 900, 7, kind="er")
    x, t = trip[:, :2].contiguous(), trip[:, 2].contiguous()
    want = m.rank_filtered(x, t, csr)
    n = len(triples)
    full = {k: torch.full((n,), -7, dtype=v.dtype, device="cuda") for k, v in want.items()}
    for i in range(0, n, 256):
        got = m.rank_filtered(x[i:i + 256], t[i:i + 256], csr, out={k: v[i:i + 256] for k, v in full.items()})
        assert got["n_greater"].data_ptr() == full["n_greater"][i:].data_ptr()
    for k in want:
        assert torch.equal(full[k], want[k]), k
    bad = dict(full)
    bad["n_equal"] = full["n_equal"].to(torch.int64)
    with pytest.raises(ValueError, match="n_equal"):
        m.rank_filtered(x, t, csr, out=bad)
    with pytest.raises(ValueError):
        m.rank_filtered(x[:10], t[:10], csr, out=full)                       # wrong length
    strided = {k: torch.empty((2 * n,), dtype=v.dtype, device="cuda")[::2] for k, v in want.items()}
    with pytest.raises(ValueError):
        m.rank_filtered(x, t, csr, out=strided)


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("QMult", 64, {})])
def test_relation_prediction_follows_the_reference_loop_literally(name, d, extra):
    """form_of_labelling='RelationPrediction' (evaluator.py:440-471): (head, tail) pairs through forward_k_vs_all,
    the (head, tail) -> relations vocabulary as the mask, the rank of column `relation` among all entity columns;
    IndexError when a tail id is not a row of the relation table."""
    from dicee_amd import Evaluator
    m, triples = _toy(name, d, n=900, seed=11, **extra)
    triples[:, 2] = triples[:, 2] % 46                     # tails that are valid relation rows
    triples[:40, [0, 2]] = triples[0, [0, 2]]              # one (head, tail) pair with many relations
    E = m.entity_embeddings.weight.detach().clone().numpy()
    Rel = m.relation_embeddings.weight.detach().clone().numpy()
    ee = {}
    for h, r, t in triples:
        ee.setdefault((int(h), int(t)), []).append(int(r))
    m = m.to("cuda")
    args = SimpleNamespace(batch_size=256, eval_model="test", scoring_technique="KvsAll", full_storage_path=None)
    # (a) the vocabulary given as the reference's dict
    ds = SimpleNamespace(num_entities=135, num_relations=46, er_vocab={}, ee_vocab=ee, train_set=triples,
                         valid_set=None, test_set=triples[200:700])
    ev = Evaluator(args)
    report = ev.eval(ds, m, "RelationPrediction", during_training=True)
    got = ev.last_ranks
    S = ko.k_vs_all_scores(name, E, Rel, triples[200:700][:, [0, 2]])
    for j, (h, r, t) in enumerate(triples[200:700]):
        tol = 1e-5 * np.sqrt((S[j] ** 2).mean())
        lo, hi = ko.rank_interval_with_tolerance(S[j], int(r), ee[(int(h), int(t))], tol)
        assert lo <= got[j] <= hi
    want = ko.relation_prediction_ranks(name, E, Rel, triples[200:700], ee)
    assert np.mean(want == got) >= 0.99
    ref = tcp.evaluate_relation_prediction(name, torch.from_numpy(E), torch.from_numpy(Rel), triples[200:700], ee, 256)
    assert np.mean(np.asarray(ref) == got) >= 0.99
    assert report["Test"]["MRR"] == pytest.approx(ko.metrics_from_ranks(got)["MRR"])
    # (b) the vocabulary built on the GPU from the dataset's splits
    ds2 = SimpleNamespace(num_entities=135, num_relations=46, train_set=triples, valid_set=None,
                          test_set=triples[200:700])
    ev2 = Evaluator(args)
    ev2.eval(ds2, m, "RelationPrediction", during_training=True)
    np.testing.assert_array_equal(ev2.last_ranks, got)
    # (c) a tail id that is not a relation row: the reference's embedding lookup raises
    bad = triples[200:210].copy()
    bad[3, 2] = 46
    with pytest.raises(IndexError):
        ev.evaluate_lp_k_vs_all(m, bad, form_of_labelling="RelationPrediction")


def test_evaluator_routes_negative_sampling_models_to_both_directions():
    """scoring_technique='NegSample' (evaluator.py:174-180, :246-272, :622-643): heads and tails through
    evaluate_lp; the report equals a direct evaluate_lp call.  'constraint' in eval_model is refused."""
    from dicee_amd import Evaluator
    from dicee_amd.link_prediction import evaluate_lp
    m, triples = _toy("ComplEx", 32, n=1200, seed=5)
    er, re = {}, {}
    for h, r, t in triples:
        er.setdefault((int(h), int(r)), []).append(int(t))
        re.setdefault((int(r), int(t)), []).append(int(h))
    m = m.to("cuda")
    ds = SimpleNamespace(num_entities=135, num_relations=46, er_vocab=er, re_vocab=re, train_set=triples,
                         valid_set=triples[:100], test_set=triples[100:500])
    ev = Evaluator(SimpleNamespace(batch_size=128, eval_model="val_test", scoring_technique="NegSample",
                                   full_storage_path=None))
    report = ev.eval(ds, m, "EntityPrediction", during_training=True)
    assert set(report) == {"Val", "Test"}
    want = evaluate_lp(m, triples[100:500], num_entities=135, er_vocab=er, re_vocab=re, info=None)
    assert report["Test"] == want
    ds2 = SimpleNamespace(num_entities=135, num_relations=46, train_set=triples, valid_set=None,
                          test_set=triples[100:500])                       # vocabularies from the splits
    ev2 = Evaluator(SimpleNamespace(batch_size=128, eval_model="test", scoring_technique="NegSample",
                                    full_storage_path=None))
    assert ev2.eval(ds2, m, "EntityPrediction", during_training=True)["Test"] == want
    ev3 = Evaluator(SimpleNamespace(batch_size=128, eval_model="test_constraint", scoring_technique="KvsAll",
                                    full_storage_path=None))
    with pytest.raises(NotImplementedError):
        ev3.eval(ds, m, "EntityPrediction", during_training=True)
    ev4 = Evaluator(SimpleNamespace(batch_size=128, eval_model=None, scoring_technique="KvsAll",
                                    full_storage_path=None))
    assert ev4.eval(ds, m, "EntityPrediction") is None


def test_predict_topk_and_predict_invariants():
    from dicee_amd import KGE
    m, _ = _toy("Keci", 32, p=0, q=1, seed=5)
    m = m.to("cuda")
    ents = [f"e{i}" for i in range(135)]
    rels = [f"r{i}" for i in range(46)]
    kge = KGE(model=m, entity_to_idx={e: i for i, e in enumerate(ents)},
              relation_to_idx={r: i for i, r in enumerate(rels)})
    # deterministic
    a = kge.predict(h=["e3"], r=["r7"])
    b = kge.predict(h=["e3"], r=["r7"])
    assert torch.equal(a, b) and a.shape == (135,)
    # top-k equals sigmoid(predict) at the same entity
    top = kge.predict_topk(h=["e3"], r=["r7"], topk=10)
    assert len(top) == 1 and len(top[0]) == 10
    probs = kge.predict(h=["e3"], r=["r7"], logits=False)
    for ent, score in top[0]:
        assert abs(probs[kge.entity_to_idx[ent]].item() - score) <= 1e-6
    scores = [s for _, s in top[0]]
    assert scores == sorted(scores, reverse=True)
    assert top[0][0][0] == ents[int(torch.argmax(probs))]
    # batch-size invariance, bitwise, heads-major cartesian order
    heads, rs = ["e1", "e9", "e30", "e77"], ["r0", "r5"]
    base = kge.predict_topk(h=heads, r=rs, topk=5, batch_size=1)
    assert len(base) == 8
    for bs in (2, 4, 8):
        assert kge.predict_topk(h=heads, r=rs, topk=5, batch_size=bs) == base
    single = kge.predict_topk(h="e9", r="r0", topk=5)
    assert single[0] == base[2]
    with pytest.raises(KeyError):
        kge.predict_topk(h=["nope"], r=["r0"])
    with pytest.raises(AttributeError):
        kge.predict_topk(h=["e1"], r=["r0"], t=["e2"])
    with pytest.raises(AssertionError):
        kge.predict_topk(h=3, r=["r0"])


@pytest.mark.parametrize("d", [32, 64, 96, 128, 192, 256, 320])   # LDS rows of 64, 128, 256 (exact and zero-padded); wider
@pytest.mark.parametrize("storage", ["bf16", "int8"])
def test_quantised_storage_follows_dequantised_fp32_math(storage, d):
    m, triples = _toy("QMult" if storage == "bf16" else "DistMult", d, N=3000, R=11, n=600, seed=7)
    m = m.to("cuda").set_entity_storage(storage)
    E, scale = m.table()
    if storage == "bf16":
        Ev = E.float().cpu().numpy()
        Rv = m._rel().float().cpu().numpy()
    else:
        Ev = (E.float() * scale[:, None]).cpu().numpy()
        Rv = m.relation_embeddings.weight.detach().cpu().numpy()
    x = torch.from_numpy(triples[:, :2].copy()).cuda()
    S = m(x).cpu().numpy()
    ref = ko.k_vs_all_scores(m.name, Ev, Rv, triples[:, :2])
    ok, worst = score_close(S, ref, 2e-2)
    assert ok, worst
    vals, idx = m.topk(x, 10)
    wv, wi = ko.topk(S, 10)
    np.testing.assert_array_equal(idx.cpu().numpy(), wi)


@pytest.mark.parametrize("storage", ["bf16", "int8"])
def test_quantised_tables_follow_the_parameters(storage):
    """The bf16 / int8 tables are copies of the parameters: after an in-place update (an optimizer step,
    load_state_dict) or a move to another device the next call scores the NEW weights."""
    from dicee_amd import ops
    m, triples = _toy("DistMult", 128, N=500, R=7, n=50, seed=9)
    m = m.set_entity_storage(storage).to("cuda").eval()             # stored on the CPU, then moved
    x = torch.from_numpy(triples[:20, :2].copy() % np.array([500, 7])).cuda()
    before = m(x).clone()
    with torch.no_grad():
        m.entity_embeddings.weight.mul_(-2.0)                        # an exact change in every storage
    after = m(x)
    # DistMult: scores are cubic in a common scale of the entity table (head row and every tail row)
    assert torch.equal(after, before * 4.0)
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    sd["entity_embeddings.weight"] = sd["entity_embeddings.weight"] * -0.5
    m.load_state_dict(sd)
    assert torch.equal(m(x), before)
    with pytest.raises(ValueError):
        ops.scores(torch.zeros((4, 64), device="cuda"), None, m.table()[0], m.table()[1])   # d mismatch: refused


def test_kvsall_bce_loss_matches_training_step_forward():
    from dicee_amd.csr import FilterCSR
    m, triples = _toy("CKeci", 64, N=2000, R=18, n=3000, seed=9, p=0, q=1)
    E = m.entity_embeddings.weight.detach().clone()
    Rel = m.relation_embeddings.weight.detach().clone()
    csr = FilterCSR.from_triples(triples, 18)
    keys = csr.keys_np[:256]
    x_np = np.stack([keys // 18, keys % 18], axis=1)
    pos = [csr.tails(int(h), int(r)) for h, r in x_np]
    m = m.to("cuda")
    csr.to("cuda")
    for eps in (0.0, 0.1):
        loss = m.kvsall_bce_loss(torch.from_numpy(x_np).cuda(), csr, eps).item()
        want = tcp.kvsall_bce_step("Keci", E, Rel, torch.from_numpy(x_np), pos, eps, p=0, q=1,
                                   coeff_q=torch.ones(1)).item()
        assert loss == pytest.approx(want, rel=2e-5)


def test_kge_from_a_dicee_experiment_folder(tmp_path):
    """model.pt / configuration.json / report.json / *_to_idx.csv round trip, then predict_topk."""
    from dicee_amd import KGE, save_experiment
    m, _ = _toy("Keci", 32, p=1, q=2, seed=11)
    ents = {f"e{i}": i for i in range(135)}
    rels = {f"r{i}": i for i in range(46)}
    save_experiment(str(tmp_path), m, ents, rels)
    kge = KGE(path=str(tmp_path))
    assert kge.model.name == "Keci" and kge.model.p == 1 and kge.model.q == 2
    assert kge.num_entities == 135 and kge.configs["num_relations"] == 46
    for k, v in m.state_dict().items():
        assert torch.equal(kge.model.state_dict()[k].cpu(), v)
    ref = KGE(model=m.to("cuda"), entity_to_idx=ents, relation_to_idx=rels)
    assert kge.predict_topk(h=["e5", "e6"], r=["r1"], topk=7) == ref.predict_topk(h=["e5", "e6"], r=["r1"], topk=7)


def test_stored_experiment_evaluates_end_to_end(tmp_path):
    """Folder with model.pt + *_set.npy (int16 ids, as dicee stores small graphs) -> report; the filter is built on
    the GPU from the stored splits and the ranks equal the oracle's on materialised fp64 scores."""
    from dicee_amd import evaluate_experiment, save_experiment
    m, triples = _toy("ComplEx", 32, n=1200, seed=13)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    splits = {"train_set": triples[:800].astype(np.int16), "valid_set": triples[800:1000].astype(np.int16),
              "test_set": triples[1000:].astype(np.int16)}
    save_experiment(str(tmp_path), m, {f"e{i}": i for i in range(135)}, {f"r{i}": i for i in range(46)},
                    extra_config={"batch_size": 128}, splits=splits)
    report, ev = evaluate_experiment(str(tmp_path), eval_model="val_test")
    assert set(report) == {"Val", "Test"} and ev.args.batch_size == 128
    keys, row_ptr, col = ko.vocab_csr(triples, "er", 46)
    np.testing.assert_array_equal(ev.csr.col.cpu().numpy(), col)
    er = ko.vocab(triples, "er")
    S = ko.k_vs_all_scores("ComplEx", E, Rel, triples[1000:, :2])
    got = ev.last_ranks                                              # of the last split evaluated: Test
    for j, (h, r, t) in enumerate(triples[1000:]):
        lo, hi = ko.rank_interval_with_tolerance(S[j], int(t), er[(int(h), int(r))], 1e-5 * np.sqrt((S[j] ** 2).mean()))
        assert lo <= got[j] <= hi
    want = ko.metrics_from_ranks(got)
    assert report["Test"]["MRR"] == pytest.approx(want["MRR"]) and report["Test"]["H@3"] == want["H@3"]


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("ComplEx", 64, {}), ("QMult", 64, {}),
                                          ("OMult", 64, {}),
                                          ("Keci", 48, {"p": 0, "q": 1}), ("Keci", 40, {"p": 2, "q": 2}),
                                          ("DeCaL", 48, {"p": 2, "q": 2, "r": 3})])
def test_evaluate_lp_both_directions(name, d, extra):
    """Head and tail ranks inside the fp64 oracle's tolerance interval, exact where there is no near-tie; metrics
    reduced as evaluate_lp does; dict and GPU-built vocabularies give the same ranks."""
    from dicee_amd import evaluate_lp, FilterCSR
    m, triples = _toy(name, d, n=1500, seed=21, **extra)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    kw = _oracle_kw(m)
    er, re = ko.vocab(triples, "er"), ko.vocab(triples, "re")
    m = m.to("cuda")
    test = triples[300:640]
    res, (hr_, tr_) = evaluate_lp(m, test, 135, er, re, info=None, batch_size=100, return_ranks=True)
    St = ko.k_vs_all_scores(name, E, Rel, test[:, :2], **kw)
    Sh = ko.all_head_scores(name, E, Rel, test[:, 1:], **kw)
    exact = 0
    for j, (h, r, t) in enumerate(test):
        h, r, t = int(h), int(r), int(t)
        lo, hi = ko.rank_interval_with_tolerance(St[j], t, er[(h, r)], 1e-5 * np.sqrt((St[j] ** 2).mean()))
        assert lo <= tr_[j] <= hi
        lo2, hi2 = ko.rank_interval_with_tolerance(Sh[j], h, re[(r, t)], 1e-5 * np.sqrt((Sh[j] ** 2).mean()))
        assert lo2 <= hr_[j] <= hi2
        exact += (lo == hi) + (lo2 == hi2)
    assert exact >= 2 * len(test) * 0.95
    want = ko.lp_metrics(hr_, tr_)
    for key in ("H@1", "H@3", "H@10", "MRR"):
        assert res[key] == pytest.approx(want[key])
    dev_trip = torch.from_numpy(triples).cuda()
    res2, (hr2, tr2) = evaluate_lp(m, test, 135, FilterCSR.from_triples_gpu(dev_trip, 135, 46, kind="er"),
                                   FilterCSR.from_triples_gpu(dev_trip, 135, 46, kind="re"), info=None,
                                   batch_size=512, return_ranks=True)
    np.testing.assert_array_equal(hr2, hr_)
    np.testing.assert_array_equal(tr2, tr_)
    assert res2 == res
    # the head-direction score matrix itself, materialised
    Sg = m.forward_all_heads(torch.from_numpy(test[:50, 1:].copy()).cuda()).cpu().numpy()
    ok, worst = score_close(Sg, Sh[:50], 1e-5)
    assert ok, worst
    with pytest.raises(AssertionError):
        evaluate_lp(m, test, 135, er, None, info=None)


def test_predict_missing_head():
    from dicee_amd import KGE
    m, _ = _toy("ComplEx", 32, seed=23)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    m = m.to("cuda")
    ents = {f"e{i}": i for i in range(135)}
    rels = {f"r{i}": i for i in range(46)}
    kge = KGE(model=m, entity_to_idx=ents, relation_to_idx=rels)
    assert not kge.all_have_inverse
    top = kge.predict_topk(r=["r3", "r4"], t=["e10", "e20", "e30"], topk=5, batch_size=4)
    assert len(top) == 6 and all(len(row) == 5 for row in top)
    # pairs are tails-major: (e10,r3), (e10,r4), (e20,r3), ...
    rt = np.array([[3, 10], [4, 10], [3, 20], [4, 20], [3, 30], [4, 30]])
    S = ko.all_head_scores("ComplEx", E, Rel, rt)
    _, wi = ko.topk(S, 5)
    for row, want_idx, srow in zip(top, wi, S):
        assert [ents[e] for e, _ in row] == want_idx.tolist()
        np.testing.assert_allclose([p for _, p in row], ko.sigmoid(srow[want_idx]), rtol=1e-5)
    full = kge.predict(r=["r3"], t=["e10"])
    assert full.shape == (135,)
    ok, worst = score_close(full.numpy()[None, :], S[:1], 1e-5)
    assert ok, worst
    assert kge.predict_topk(r="r3", t="e10", topk=5)[0] == top[0]
    # missing relation: every (h, x, t) scored as a triple
    rel_top = kge.predict_topk(h=["e1", "e5"], t=["e2"], topk=3)
    trip = np.array([[hh, x, 2] for hh in (1, 5) for x in range(46)])
    ref_r = ko.triple_scores("ComplEx", E, Rel, trip).reshape(2, 46)
    for row, want_row in zip(rel_top, ref_r):
        order = np.argsort(-want_row, kind="stable")[:3]
        assert [rels[name] for name, _ in row] == order.tolist()
        np.testing.assert_allclose([p for _, p in row], ko.sigmoid(want_row[order]), rtol=1e-5)
    assert kge.predict(h=["e1"], t=["e2"]).shape == (46,)
    # reciprocal vocabulary: the head question is asked as a tail question with r_inverse
    rels2 = {f"r{i}": i for i in range(23)}
    rels2.update({f"r{i}_inverse": 23 + i for i in range(23)})
    kge2 = KGE(model=m, entity_to_idx=ents, relation_to_idx=rels2)
    assert kge2.all_have_inverse
    assert kge2.predict_topk(r=["r3"], t=["e10"], topk=4) == kge2.predict_topk(h=["e10"], r=["r3_inverse"], topk=4)


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("ComplEx", 32, {}), ("QMult", 32, {}),
                                          ("Keci", 30, {"p": 2, "q": 2}), ("DeCaL", 32, {"p": 2, "q": 2, "r": 3})])
def test_forward_triples_and_triple_score(name, d, extra):
    from dicee_amd import KGE
    m, triples = _toy(name, d, n=400, seed=31, **extra)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    kw = _oracle_kw(m)
    m = m.to("cuda").eval()
    x = torch.from_numpy(triples).cuda()
    with torch.no_grad():
        s = m(x)                                                   # three columns -> forward_triples
    assert s.shape == (400,) and s.dtype == torch.float32
    ref = ko.triple_scores(name, E, Rel, triples, **kw)
    assert np.abs(s.cpu().numpy() - ref).max() <= 1e-5 * np.sqrt((ref ** 2).mean()) + 1e-7
    # the same bits as the matching column of the KvsAll scores
    S = m(x[:, :2].contiguous())
    assert torch.equal(S[torch.arange(400), x[:, 2]], s)
    ents = {f"e{i}": i for i in range(135)}
    rels = {f"r{i}": i for i in range(46)}
    kge = KGE(model=m, entity_to_idx=ents, relation_to_idx=rels)
    h, r, t = (int(v) for v in triples[7])
    one = kge.triple_score(f"e{h}", f"r{r}", f"e{t}")
    assert one.shape == (1,) and abs(float(one) - float(ko.sigmoid(ref[7:8])[0])) <= 1e-6
    many = kge.triple_score([f"e{a}" for a in triples[:5, 0]], [f"r{a}" for a in triples[:5, 1]],
                            [f"e{a}" for a in triples[:5, 2]], logits=True)
    assert torch.equal(many, s[:5])
    assert torch.allclose(kge.predict(h=[f"e{h}"], r=[f"r{r}"], t=[f"e{t}"]), s[7:8].cpu())
    with pytest.raises(KeyError):
        kge.triple_score("nobody", "r0", "e1")


@pytest.mark.parametrize("kind", ["LayerNorm", "BatchNorm1d"])
def test_forward_triples_normalises_the_tail_of_a_model_trained_on_single_triples(kind):
    """normalization + NegSample / KvsSample: the reference also normalises the tail row (base_model.py:287-294,
    :374); the module exists (so a stored state_dict loads strictly) and forward_triples applies it."""
    from dicee_amd import evaluate_lp
    d = 32
    m, triples = _toy("DistMult", d, n=300, seed=41, normalization=kind, scoring_technique="NegSample")
    assert any(k.startswith("normalize_tail_entity_embeddings.") for k in m.state_dict())
    rng = np.random.default_rng(3)
    with torch.no_grad():
        for mod in (m.normalize_head_entity_embeddings, m.normalize_relation_embeddings, m.normalize_tail_entity_embeddings):
            if kind == "LayerNorm":
                mod.weight.copy_(torch.from_numpy(rng.normal(1.0, 0.2, d).astype(np.float32)))
                mod.bias.copy_(torch.from_numpy(rng.normal(0.0, 0.1, d).astype(np.float32)))
            else:
                mod.running_mean.copy_(torch.from_numpy(rng.normal(0.0, 0.05, d).astype(np.float32)))
                mod.running_var.copy_(torch.from_numpy(rng.uniform(0.5, 1.5, d).astype(np.float32)))
    E = m.entity_embeddings.weight.detach().numpy().astype(np.float64)
    Rel = m.relation_embeddings.weight.detach().numpy().astype(np.float64)

    def normed(mod, x):
        if kind == "LayerNorm":
            return ko.layer_norm(x, mod.weight.detach().numpy(), mod.bias.detach().numpy(), mod.eps)
        return ko.batch_norm_eval(x, mod.running_mean.numpy(), mod.running_var.numpy(), mod.eps)
    h = normed(m.normalize_head_entity_embeddings, E[triples[:, 0]])
    r = normed(m.normalize_relation_embeddings, Rel[triples[:, 1]])
    t = normed(m.normalize_tail_entity_embeddings, E[triples[:, 2]])
    ref = (h * r * t).sum(axis=1)
    m = m.to("cuda").eval()
    with torch.no_grad():
        s = m(torch.from_numpy(triples).cuda())
    assert s.shape == (300,)
    assert np.abs(s.cpu().numpy() - ref).max() <= 1e-5 * np.sqrt((ref ** 2).mean()) + 1e-6
    # a model without the tail normaliser (KvsAll-trained) keeps scoring against the table as it is
    m2, _ = _toy("DistMult", d, n=10, seed=41, normalization=kind, scoring_technique="KvsAll")
    assert not any(k.startswith("normalize_tail_entity_embeddings.") for k in m2.state_dict())
    # ranking against the un-normalised table would be silently wrong for such a model: refused
    with pytest.raises(NotImplementedError):
        evaluate_lp(m, triples, er_vocab={}, re_vocab={}, info=None)
    with pytest.raises(IndexError):
        m(torch.tensor([[0, 0, 135]]).cuda())


def test_string_triple_evaluators():
    from dicee_amd import (KGE, evaluate_lp, evaluate_link_prediction_performance,
                           evaluate_link_prediction_performance_with_reciprocals)
    m, triples = _toy("ComplEx", 32, n=900, seed=33, batch_size=64)
    ents = {f"e{i}": i for i in range(135)}
    rels = {f"r{i}": i for i in range(46)}
    m = m.to("cuda")
    kge = KGE(model=m, entity_to_idx=ents, relation_to_idx=rels)
    strs = [(f"e{h}", f"r{r}", f"e{t}") for h, r, t in triples]
    er_s, re_s = {}, {}
    for h, r, t in strs:
        er_s.setdefault((h, r), []).append(t)
        re_s.setdefault((r, t), []).append(h)
    test = strs[600:]
    both = evaluate_link_prediction_performance(kge, test, er_s, re_s)
    want = evaluate_lp(m, triples[600:], 135, ko.vocab(triples, "er"), ko.vocab(triples, "re"), info=None, batch_size=64)
    assert both == want
    tails = evaluate_link_prediction_performance_with_reciprocals(kge, test, er_s)
    from dicee_amd import Evaluator
    ev = Evaluator(SimpleNamespace(batch_size=64, eval_model="test", scoring_technique="KvsAll", full_storage_path=None))
    ev.set_filter(ko.vocab(triples, "er"), 46)
    want_t = ev.evaluate_lp_k_vs_all(m, triples[600:])
    assert set(tails) == {"H@1", "H@3", "H@10", "MRR"}
    for key in tails:
        assert tails[key] == pytest.approx(want_t[key])
    with pytest.raises(KeyError):
        evaluate_link_prediction_performance_with_reciprocals(kge, [("e1", "r1", "stranger")], er_s)


@pytest.mark.parametrize("normalize,weighted", [(True, True), (True, False), (False, True)])
def test_ensemble_evaluation(normalize, weighted):
    from dicee_amd import evaluate_ensemble_link_prediction_performance as ens_eval
    from dicee_amd import ops
    members = [_toy("DistMult", 32, n=1200, seed=41), _toy("ComplEx", 64, n=1200, seed=42),
               _toy("Keci", 30, n=1200, seed=43, p=2, q=2)]
    triples = members[0][1]
    er = ko.vocab(triples, "er")
    test = triples[700:1000]
    weights = [0.5, 0.3, 0.2]
    S = []
    for (m, _), name in zip(members, ("DistMult", "ComplEx", "Keci")):
        S.append(ko.k_vs_all_scores(name, m.entity_embeddings.weight.detach().numpy(),
                                    m.relation_embeddings.weight.detach().numpy(), test[:, :2], **_oracle_kw(m)))
    want = ko.ensemble_scores(S, weights, weighted, normalize)
    gpu_models = [m.to("cuda") for m, _ in members]
    # the fused row extrema against the oracle's
    x = torch.from_numpy(test[:, :2].copy()).cuda()
    Q, bias = gpu_models[1].query(x)
    lo, hi = ops.row_minmax(Q, bias, *gpu_models[1].table())
    assert np.abs(lo.cpu().numpy() - S[1].min(1)).max() <= 1e-5 * np.abs(S[1]).max()
    assert np.abs(hi.cpu().numpy() - S[1].max(1)).max() <= 1e-5 * np.abs(S[1]).max()
    res, ranks = ens_eval(gpu_models, test, er, weights=weights if weighted else None, batch_size=128,
                          weighted_averaging=weighted, normalize_scores=normalize, return_ranks=True)
    exact = 0
    for j, (h, r, t) in enumerate(test):
        tol = 2e-5 * (1.0 if normalize else np.sqrt((want[j] ** 2).mean()))
        lo_r, hi_r = ko.rank_interval_with_tolerance(want[j], int(t), er[(int(h), int(r))], tol)
        assert lo_r <= ranks[j] <= hi_r
        exact += lo_r == hi_r
    assert exact >= 0.9 * len(test)
    wm = ko.metrics_from_ranks(ranks)
    assert res["MRR"] == pytest.approx(wm["MRR"]) and res["H@10"] == wm["H@10"]
    if weighted:
        with pytest.raises(AssertionError):
            ens_eval(gpu_models, test, er, weights=[1.0], weighted_averaging=True)


def test_multi_hop_queries_against_the_oracle():
    from dicee_amd import KGE
    m, triples = _toy("ComplEx", 32, seed=51)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    m = m.to("cuda")
    ents = {f"e{i}": i for i in range(135)}
    rels = {f"r{i}": i for i in range(46)}
    kge = KGE(model=m, entity_to_idx=ents, relation_to_idx=rels)
    atom = lambda heads, r: ko.k_vs_all_scores("ComplEx", E, Rel, np.array([[h, r] for h in heads]))
    n = lambda q: q                                        # readability: queries are given with names
    cases = [
        ("1p", ("e3", ("r1",)), (3, (1,))),
        ("2p", ("e3", ("r1", "r4")), (3, (1, 4))),
        ("3p", ("e3", ("r1", "r4", "r9")), (3, (1, 4, 9))),
        ("2i", (("e3", ("r1",)), ("e8", ("r2",))), ((3, (1,)), (8, (2,)))),
        ("3i", (("e3", ("r1",)), ("e8", ("r2",)), ("e11", ("r5",))), ((3, (1,)), (8, (2,)), (11, (5,)))),
        ("ip", ((("e3", ("r1",)), ("e8", ("r2",))), ("r7",)), (((3, (1,)), (8, (2,))), (7,))),
        ("pi", (("e3", ("r1", "r4")), ("e8", ("r2",))), ((3, (1, 4)), (8, (2,)))),
        ("2in", (("e3", ("r1",)), ("e8", ("r2", "n"))), ((3, (1,)), (8, (2, "n")))),
        ("3in", (("e3", ("r1",)), ("e8", ("r2",)), ("e11", ("r5", "n"))), ((3, (1,)), (8, (2,)), (11, (5, "n")))),
        ("inp", ((("e3", ("r1",)), ("e8", ("r2", "n"))), ("r7",)), (((3, (1,)), (8, (2, "n"))), (7,))),
        ("pin", (("e3", ("r1", "r4")), ("e8", ("r2", "n"))), ((3, (1, 4)), (8, (2, "n")))),
        ("pni", (("e3", ("r1", "r4", "n")), ("e8", ("r2",))), ((3, (1, 4, "n")), (8, (2,)))),
        ("2u", (("e3", ("r1",)), ("e8", ("r2",)), ("u",)), ((3, (1,)), (8, (2,)), ("u",))),
        ("up", ((("e3", ("r1",)), ("e8", ("r2",)), ("u",)), ("r7",)), (((3, (1,)), (8, (2,)), ("u",)), (7,))),
    ]
    for tnorm in ("min", "prod"):
        for qtype, q_named, q_ids in cases:
            got = kge.answer_multi_hop_query(query_type=qtype, query=n(q_named), tnorm=tnorm, k=5, only_scores=True)
            want = ko.multi_hop_scores(atom, qtype, q_ids, tnorm=tnorm, k=5)
            assert got.shape == (135,)
            np.testing.assert_allclose(got.numpy(), want, rtol=2e-4, atol=2e-5, err_msg=f"{qtype} {tnorm}")
    top = kge.answer_multi_hop_query(query_type="2p", query=("e3", ("r1", "r4")), tnorm="min", k=5)
    assert len(top) == 5 and [s for _, s in top] == sorted((s for _, s in top), reverse=True)
    want = ko.multi_hop_scores(atom, "2p", (3, (1, 4)), tnorm="min", k=5)
    assert top[0][0] == f"e{int(np.argmax(want))}"
    full = kge.answer_multi_hop_query(query_type="2i", query=(("e3", ("r1",)), ("e8", ("r2",))), tnorm="min")
    assert len(full) == 135
    both = kge.answer_multi_hop_query(query_type="1p", queries=[("e3", ("r1",)), ("e4", ("r2",))], only_scores=True)
    assert len(both) == 2 and torch.equal(both[0], kge.predict(h=["e3"], r=["r1"]))
    with pytest.raises(ValueError):
        kge.answer_multi_hop_query(query_type="4p", query=("e3", ("r1",)))


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("Keci", 30, {"p": 2, "q": 2}),
                                          ("DeCaL", 32, {"p": 2, "q": 2, "r": 3})])
def test_kvsall_bce_backward_through_the_model(name, d, extra):
    """Loss and gradients of the KvsAll BCE step at the query vectors, the per-query biases and the entity table,
    against the fp64 closed form on the oracle's query vectors."""
    from dicee_amd import FilterCSR
    m, triples = _toy(name, d, n=900, seed=51, **extra)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    kw = _oracle_kw(m)
    er = ko.vocab(triples, "er")
    m = m.to("cuda").eval()
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    x_np = triples[:300, :2]
    loss, dQ, dbias, dE = m.kvsall_bce_backward(torch.from_numpy(x_np.copy()).cuda(), csr, label_smoothing=0.1)
    Qr, br = ko.build_query(name, E, Rel, x_np, **kw)
    positives = [er[(int(h), int(r))] for h, r in x_np]
    want_loss = ko.bce_multihot(Qr @ E.T + br[:, None], positives, 0.1)
    assert loss.item() == pytest.approx(want_loss, rel=1e-5)
    wQ, wb, wE = ko.bce_multihot_backward(Qr, br, E, positives, 0.1)
    for got, want in ((dQ, wQ), (dE, wE)):
        assert np.abs(got.cpu().numpy() - want).max() <= 1e-5 * np.sqrt((want ** 2).mean())
    g_abs = (ko.sigmoid(Qr @ E.T + br[:, None]) + ko.dense_multihot(positives, 135, 0.1, dtype=np.float64)) / (300 * 135)
    assert np.all(np.abs(dbias.cpu().numpy() - wb) <= 2e-6 * g_abs.sum(axis=1))
    m.set_entity_storage("bf16")
    with pytest.raises(TypeError):
        m.kvsall_bce_backward(torch.from_numpy(x_np.copy()).cuda(), csr)


def test_rank_bce_and_backward_steps_replay_from_a_hip_graph():
    """The entry points that neither allocate nor synchronise can be captured into a HIP graph by the caller: the
    filtered-rank step, the BCE loss and its backward, replayed several times with eager work of the same library
    between the replays, give the eager results every time (dbias: summed with atomics, so only to rounding)."""
    from dicee_amd import FilterCSR
    m, triples = _toy("Keci", 30, n=1200, seed=61, p=2, q=2)
    er = ko.vocab(triples, "er")
    m = m.to("cuda").eval()
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    x = torch.from_numpy(triples[:400, :2].copy()).cuda()
    t = torch.from_numpy(triples[:400, 2].copy()).cuda()

    def step():
        r = m.rank_filtered(x, t, csr)
        loss, dQ, dbias, dE = m.kvsall_bce_backward(x, csr, label_smoothing=0.1)
        return r, m.kvsall_bce_loss(x, csr), loss, dQ, dbias, dE

    eager = step()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()                                                # warm-up on a side stream, as capture requires
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        for key in eager[0]:
            assert torch.equal(captured[0][key], eager[0][key]), key
        assert torch.equal(captured[1], eager[1]) or captured[1].item() == pytest.approx(eager[1].item(), rel=1e-6)
        assert captured[2].item() == pytest.approx(eager[2].item(), rel=1e-6)
        assert torch.equal(captured[3], eager[3]) and torch.equal(captured[5], eager[5])
        assert (captured[4] - eager[4]).abs().max().item() <= 1e-6 * eager[4].abs().max().item() + 1e-12
        step()                                                    # eager work between replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("ComplEx", 32, {}), ("QMult", 32, {}),
                                          ("Keci", 30, {"p": 2, "q": 2})])
def test_full_step_gradients_match_autograd_through_the_reference_op_sequence(name, d, extra):
    """loss and every parameter gradient of one KvsAll BCE training step against torch autograd (float64, CPU)
    through the reference's own op sequence: embedding lookups, the model's k_vs_all_score, BCEWithLogitsLoss on
    the dense smoothed multi-hot target."""
    from dicee_amd import FilterCSR
    m, triples = _toy(name, d, n=900, seed=71, **extra)
    er = ko.vocab(triples, "er")
    kw = _oracle_kw(m)
    E = m.entity_embeddings.weight.detach().double().clone().requires_grad_()
    Rel = m.relation_embeddings.weight.detach().double().clone().requires_grad_()
    tkw = {k: (torch.tensor(v, dtype=torch.float64, requires_grad=True) if k.startswith("coeff") else v)
           for k, v in kw.items()}
    x_np = triples[:256, :2]
    positives = [er[(int(h), int(r))] for h, r in x_np]
    ref = tcp.kvsall_bce_step(name, E, Rel, torch.from_numpy(x_np.copy()), positives, 0.1, **tkw)
    ref.backward()
    m = m.to("cuda").eval()
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    loss, grads = m.kvsall_bce_gradients(torch.from_numpy(x_np.copy()).cuda(), csr, label_smoothing=0.1)
    assert loss.item() == pytest.approx(ref.item(), rel=1e-5)
    want = {"entity_embeddings.weight": E.grad, "relation_embeddings.weight": Rel.grad}
    if "coeff_p" in tkw:
        want["p_coefficients.weight"] = tkw["coeff_p"].grad.reshape(1, -1)
    if "coeff_q" in tkw:
        want["q_coefficients.weight"] = tkw["coeff_q"].grad.reshape(1, -1)
    assert set(grads) == set(want)
    for key, w in want.items():
        w = w.numpy()
        g = grads[key].cpu().numpy()
        assert g.shape == w.shape, key
        rms = np.sqrt((w ** 2).mean())
        assert np.abs(g - w).max() <= 3e-5 * rms + 1e-9, (key, np.abs(g - w).max() / rms)


@pytest.mark.parametrize("name,d,extra,kind", [("DistMult", 32, {}, "LayerNorm"), ("QMult", 32, {}, "LayerNorm"),
                                               ("Keci", 30, {"p": 2, "q": 2}, "LayerNorm"),
                                               ("ComplEx", 32, {}, "BatchNorm1d")])
def test_full_step_gradients_through_the_normalisation_layer_match_autograd(name, d, extra, kind):
    """The same with ``normalization='LayerNorm'`` (in training mode: the layer has no other mode; its weights and
    biases receive gradients too) and ``'BatchNorm1d'`` in eval mode (running statistics), against autograd through
    torch's own modules placed where base_model.py:381-383 places them."""
    from dicee_amd import FilterCSR
    m, triples = _toy(name, d, n=900, seed=75, normalization=kind, **extra)
    rng = np.random.default_rng(5)
    with torch.no_grad():
        for mod in (m.normalize_head_entity_embeddings, m.normalize_relation_embeddings):
            if kind == "LayerNorm":
                mod.weight.copy_(torch.from_numpy(rng.uniform(0.5, 1.5, d).astype(np.float32)))
                mod.bias.copy_(torch.from_numpy(rng.normal(0, 0.2, d).astype(np.float32)))
            else:
                mod.running_mean.copy_(torch.from_numpy(rng.normal(0, 0.05, d).astype(np.float32)))
                mod.running_var.copy_(torch.from_numpy(rng.uniform(0.005, 0.02, d).astype(np.float32)))
    er = ko.vocab(triples, "er")
    kw = _oracle_kw(m)
    if name == "QMult":
        kw["normalize_relation"] = False          # quaternion.py:138: only without another relation normaliser
    E = m.entity_embeddings.weight.detach().double().clone().requires_grad_()
    Rel = m.relation_embeddings.weight.detach().double().clone().requires_grad_()
    tkw = {k: (torch.tensor(v, dtype=torch.float64, requires_grad=True) if k.startswith("coeff") else v)
           for k, v in kw.items()}
    import copy
    ref_h = copy.deepcopy(m.normalize_head_entity_embeddings).double()
    ref_r = copy.deepcopy(m.normalize_relation_embeddings).double()
    if kind == "BatchNorm1d":
        ref_h.eval(), ref_r.eval()
    x_np = triples[:256, :2]
    positives = [er[(int(h), int(r))] for h, r in x_np]
    ref = tcp.kvsall_bce_step(name, E, Rel, torch.from_numpy(x_np.copy()), positives, 0.1, norm_h=ref_h, norm_r=ref_r,
                              **tkw)
    ref.backward()
    m = m.to("cuda")
    m = m.train() if kind == "LayerNorm" else m.eval()
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    loss, grads = m.kvsall_bce_gradients(torch.from_numpy(x_np.copy()).cuda(), csr, label_smoothing=0.1)
    assert loss.item() == pytest.approx(ref.item(), rel=1e-5)
    want = {"entity_embeddings.weight": E.grad, "relation_embeddings.weight": Rel.grad}
    if "coeff_p" in tkw:
        want["p_coefficients.weight"] = tkw["coeff_p"].grad.reshape(1, -1)
    if "coeff_q" in tkw:
        want["q_coefficients.weight"] = tkw["coeff_q"].grad.reshape(1, -1)
    if kind == "LayerNorm":
        want["normalize_head_entity_embeddings.weight"] = ref_h.weight.grad
        want["normalize_head_entity_embeddings.bias"] = ref_h.bias.grad
        want["normalize_relation_embeddings.weight"] = ref_r.weight.grad
        want["normalize_relation_embeddings.bias"] = ref_r.bias.grad
    assert set(grads) == set(want)
    for key, w in want.items():
        w = w.numpy()
        g = grads[key].cpu().numpy()
        assert g.shape == w.shape, key
        rms = np.sqrt((w ** 2).mean())
        assert np.abs(g - w).max() <= 5e-5 * rms + 1e-9, (key, np.abs(g - w).max() / rms)


@pytest.mark.parametrize("name,d,extra", [("DistMult", 32, {}), ("Keci", 30, {"p": 2, "q": 2}),
                                          ("ComplEx", 32, {"normalization": "LayerNorm"}),
                                          ("QMult", 32, {"normalization": "BatchNorm1d"})])
def test_full_step_in_training_mode_with_dropout_matches_autograd_given_the_masks_it_drew(name, d, extra):
    """input_dropout_rate = 0.3, model.train(): the step draws its masks from torch's generator; with those masks
    placed where the reference places its Dropout modules (base_model.py:381-383, real.py:32) autograd gives the same
    loss and gradients.  Eval mode draws nothing and is unaffected."""
    from dicee_amd import FilterCSR
    import copy
    m, triples = _toy(name, d, n=900, seed=79, input_dropout_rate=0.3, **extra)
    er = ko.vocab(triples, "er")
    kw = _oracle_kw(m)
    if name == "QMult":
        kw["normalize_relation"] = False
    E = m.entity_embeddings.weight.detach().double().clone().requires_grad_()
    Rel = m.relation_embeddings.weight.detach().double().clone().requires_grad_()
    tkw = {k: (torch.tensor(v, dtype=torch.float64, requires_grad=True) if k.startswith("coeff") else v)
           for k, v in kw.items()}
    ref_h = copy.deepcopy(m.normalize_head_entity_embeddings).double().train()
    ref_r = copy.deepcopy(m.normalize_relation_embeddings).double().train()
    x_np = triples[:256, :2]
    positives = [er[(int(h), int(r))] for h, r in x_np]
    m = m.to("cuda").train()
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    drawn = []
    draw = m._draw_dropout
    m._draw_dropout = lambda *a, **k: drawn.append(draw(*a, **k)) or drawn[-1]
    torch.manual_seed(123)
    loss, grads = m.kvsall_bce_gradients(torch.from_numpy(x_np.copy()).cuda(), csr, label_smoothing=0.1)
    assert len(drawn) == 1                     # one set of masks for the forward and the backward of the step
    drop = drawn[0]
    scale = 1 / 0.7
    kh, kr = drop["keep_h"].cpu().double(), drop["keep_r"].cpu().double()
    assert 0.6 < float(kh.mean()) < 0.8 and not torch.equal(kh, kr)
    hidden = None
    if name == "DistMult":
        kq = drop["keep_q"].cpu().double()
        hidden = lambda v: v * kq * scale      # noqa: E731
    else:
        assert "keep_q" not in drop
    ref = tcp.kvsall_bce_step(name, E, Rel, torch.from_numpy(x_np.copy()), positives, 0.1,
                              norm_h=lambda rows: ref_h(rows * kh * scale), norm_r=lambda rows: ref_r(rows * kr * scale),
                              **({"hidden": hidden} if hidden else {}), **tkw)
    ref.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-5)
    want = {"entity_embeddings.weight": E.grad, "relation_embeddings.weight": Rel.grad}
    if "coeff_p" in tkw:
        want["p_coefficients.weight"] = tkw["coeff_p"].grad.reshape(1, -1)
        want["q_coefficients.weight"] = tkw["coeff_q"].grad.reshape(1, -1)
    if extra.get("normalization") == "LayerNorm":
        want["normalize_head_entity_embeddings.weight"] = ref_h.weight.grad
        want["normalize_head_entity_embeddings.bias"] = ref_h.bias.grad
        want["normalize_relation_embeddings.weight"] = ref_r.weight.grad
        want["normalize_relation_embeddings.bias"] = ref_r.bias.grad
    assert set(grads) == set(want)
    for key, w in want.items():
        w = w.numpy()
        g = grads[key].cpu().numpy()
        rms = np.sqrt((w ** 2).mean())
        assert np.abs(g - w).max() <= 1e-4 * rms + 1e-9, (key, np.abs(g - w).max() / rms)
    # a second step draws other masks; eval mode draws none and scores as a model without dropout
    m.kvsall_bce_gradients(torch.from_numpy(x_np.copy()).cuda(), csr)
    assert len(drawn) == 2 and not torch.equal(drawn[0]["keep_h"], drawn[1]["keep_h"])
    m.eval()
    s1 = m(torch.from_numpy(x_np[:4].copy()).cuda())
    s2 = m(torch.from_numpy(x_np[:4].copy()).cuda())
    assert torch.equal(s1, s2) and drawn[-1] is None


def test_full_step_in_training_mode_with_batchnorm_matches_torch_modules_in_training_mode():
    """normalization='BatchNorm1d', model.train(): loss, gradients and the running statistics the step leaves against
    torch.nn.BatchNorm1d(affine=False).train() modules inside the reference's op sequence (float64, CPU)."""
    from dicee_amd import FilterCSR
    import copy
    d = 32
    m, triples = _toy("ComplEx", d, n=900, seed=77, normalization="BatchNorm1d")
    er = ko.vocab(triples, "er")
    E = m.entity_embeddings.weight.detach().double().clone().requires_grad_()
    Rel = m.relation_embeddings.weight.detach().double().clone().requires_grad_()
    ref_h = copy.deepcopy(m.normalize_head_entity_embeddings).double().train()
    ref_r = copy.deepcopy(m.normalize_relation_embeddings).double().train()
    x_np = triples[:256, :2]
    positives = [er[(int(h), int(r))] for h, r in x_np]
    ref = tcp.kvsall_bce_step("ComplEx", E, Rel, torch.from_numpy(x_np.copy()), positives, 0.1, norm_h=ref_h, norm_r=ref_r)
    ref.backward()
    m = m.to("cuda").train()
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    loss, grads = m.kvsall_bce_gradients(torch.from_numpy(x_np.copy()).cuda(), csr, label_smoothing=0.1)
    assert loss.item() == pytest.approx(ref.item(), rel=1e-5)
    want = {"entity_embeddings.weight": E.grad, "relation_embeddings.weight": Rel.grad}
    assert set(grads) == set(want)
    for key, w in want.items():
        w = w.numpy()
        g = grads[key].cpu().numpy()
        rms = np.sqrt((w ** 2).mean())
        assert np.abs(g - w).max() <= 1e-4 * rms + 1e-9, (key, np.abs(g - w).max() / rms)
    for ours, theirs in ((m.normalize_head_entity_embeddings, ref_h), (m.normalize_relation_embeddings, ref_r)):
        assert int(ours.num_batches_tracked) == int(theirs.num_batches_tracked) == 1
        np.testing.assert_allclose(ours.running_mean.cpu().numpy(), theirs.running_mean.numpy(), rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(ours.running_var.cpu().numpy(), theirs.running_var.numpy(), rtol=1e-5, atol=1e-7)
    # eval mode afterwards scores with the running statistics, as the module does
    m.eval()
    s = m(torch.from_numpy(x_np[:8].copy()).cuda()).cpu().numpy()
    with torch.no_grad():
        want_s = tcp.forward_k_vs_all("ComplEx", E.detach(), Rel.detach(), torch.from_numpy(x_np[:8].copy()),
                                      norm_h=ref_h.eval(), norm_r=ref_r.eval()).numpy()
    ok, worst = score_close(s, want_s, 1e-4)
    assert ok, worst


def test_full_step_gradients_of_omult_and_decal_against_the_composed_oracle():
    from dicee_amd import FilterCSR
    for name, d, extra in (("OMult", 32, {}), ("DeCaL", 32, {"p": 2, "q": 2, "r": 3})):
        m, triples = _toy(name, d, n=900, seed=73, **extra)
        E = m.entity_embeddings.weight.detach().numpy().astype(np.float64)
        Rel = m.relation_embeddings.weight.detach().numpy().astype(np.float64)
        kw = _oracle_kw(m)
        er = ko.vocab(triples, "er")
        x_np = triples[:200, :2]
        positives = [er[(int(h), int(r))] for h, r in x_np]
        Qr, br = ko.build_query(name, E, Rel, x_np, **kw)
        dQ, dbias, dE = ko.bce_multihot_backward(Qr, br, E, positives, 0.1)
        dE2, dR, dc = ko.build_query_backward(name, E, Rel, x_np, dQ, dbias, **kw)
        m = m.to("cuda").eval()
        csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
        loss, grads = m.kvsall_bce_gradients(torch.from_numpy(x_np.copy()).cuda(), csr, label_smoothing=0.1)
        want = {"entity_embeddings.weight": dE + dE2, "relation_embeddings.weight": dR}
        for key, attr in (("coeff_p", "p_coefficients.weight"), ("coeff_q", "q_coefficients.weight"),
                          ("coeff_r", "r_coefficients.weight")):
            if key in dc:
                want[attr] = dc[key].reshape(1, -1)
        assert set(grads) == set(want)
        for key, w in want.items():
            g = grads[key].cpu().numpy()
            rms = np.sqrt((w ** 2).mean())
            assert np.abs(g - w).max() <= 3e-5 * rms + 1e-9, (name, key, np.abs(g - w).max() / rms)


def test_a_few_optimizer_steps_track_the_reference_training_loop():
    """Ten Adam steps on a small Keci model: losses from the fused step + torch.optim on the GPU against the
    reference's op sequence with autograd on the CPU (float64), same initial weights and batches."""
    from dicee_amd import FilterCSR
    m, triples = _toy("Keci", 30, n=1500, seed=81, p=2, q=2)
    er = ko.vocab(triples, "er")
    E = m.entity_embeddings.weight.detach().double().clone().requires_grad_()
    Rel = m.relation_embeddings.weight.detach().double().clone().requires_grad_()
    cp = m.p_coefficients.weight.detach().double().reshape(-1).clone().requires_grad_()
    cq = m.q_coefficients.weight.detach().double().reshape(-1).clone().requires_grad_()
    ref_opt = torch.optim.Adam([E, Rel, cp, cq], lr=0.05)
    m = m.to("cuda").train()
    for prm in m.parameters():
        prm.requires_grad_(True)
    opt = torch.optim.Adam(m.parameters(), lr=0.05)
    csr = FilterCSR.from_er_vocab(er, 46, device="cuda")
    ours, theirs = [], []
    for step in range(10):
        x_np = triples[step * 128:(step + 1) * 128, :2]
        positives = [er[(int(h), int(r))] for h, r in x_np]
        ref_opt.zero_grad()
        ref = tcp.kvsall_bce_step("Keci", E, Rel, torch.from_numpy(x_np.copy()), positives, 0.0, p=2, q=2,
                                  coeff_p=cp, coeff_q=cq)
        ref.backward()
        ref_opt.step()
        theirs.append(ref.item())
        opt.zero_grad(set_to_none=True)
        loss = m.kvsall_training_step(torch.from_numpy(x_np.copy()).cuda(), csr)
        opt.step()
        ours.append(loss.item())
    assert theirs[-1] < theirs[0]
    np.testing.assert_allclose(ours, theirs, rtol=2e-4)
    np.testing.assert_allclose(m.entity_embeddings.weight.detach().cpu().numpy(), E.detach().numpy(), atol=2e-3)


@pytest.mark.parametrize("name,d,extra,storage", [("DistMult", 32, {}, "fp32"), ("ComplEx", 32, {}, "fp32"),
                                                  ("QMult", 32, {}, "fp32"), ("Keci", 30, {"p": 2, "q": 2}, "fp32"),
                                                  ("QMult", 128, {}, "bf16"), ("DistMult", 128, {}, "int8")])
def test_forward_k_vs_sample_is_the_sampled_columns_of_kvsall(name, d, extra, storage):
    """BaseKGE.forward on a tuple (x, target_entity_idx): [B,k] scores equal, bit for bit, to the sampled columns
    of the model's own KvsAll scores, and within tolerance of the oracle."""
    m, triples = _toy(name, d, n=400, seed=91, **extra)
    E = m.entity_embeddings.weight.detach().numpy().copy()
    Rel = m.relation_embeddings.weight.detach().numpy().copy()
    kw = _oracle_kw(m)
    m = m.to("cuda").eval()
    m.set_entity_storage(storage)
    rng = np.random.default_rng(5)
    x = torch.from_numpy(triples[:150, :2].copy()).cuda()
    idx = torch.from_numpy(rng.integers(0, 135, (150, 7))).cuda()
    with torch.no_grad():
        out = m((x, idx))
        full = m(x)
    assert out.shape == (150, 7) and out.dtype == torch.float32
    assert torch.equal(out, torch.gather(full, 1, idx))
    if storage == "fp32":
        ref = ko.k_vs_all_scores(name, E, Rel, triples[:150, :2], **kw)
        want = np.take_along_axis(ref, idx.cpu().numpy(), axis=1)
        assert np.abs(out.cpu().numpy() - want).max() <= 1e-5 * np.sqrt((ref ** 2).mean()) + 1e-7
    bad = idx.clone()
    bad[0, 0] = 135
    assert torch.isnan(m((x, bad))[0, 0])
