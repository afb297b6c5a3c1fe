"""CPU-only checks: host-side logic of the package, and that the C-ABI library loads and exports
every symbol ``include/kge_hip.h`` declares (no kernel is launched here)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import kge_oracle as ko

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib_path():
    from dicee_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build()
    return _lib.LIB_PATH


def test_library_exports_every_declared_symbol(lib_path):
    header = open(os.path.join(ROOT, "include", "kge_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = sorted(set(re.findall(r"\b(kge_[a-z_0-9]+)\s*\(", header)))
    assert {"kge_build_query", "kge_scores", "kge_rank_filtered", "kge_topk", "kge_bce_multihot",
            "kge_last_error", "kge_abi_version", "kge_rank_workspace_bytes", "kge_topk_workspace_bytes",
            "kge_bce_workspace_bytes"} <= set(declared)
    lib = ctypes.CDLL(lib_path)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in kge_hip.h but not exported"
    from dicee_amd import _lib
    assert set(_lib.SIGNATURES) == set(declared)
    loaded = _lib.load()
    assert loaded.kge_abi_version() == 1
    assert loaded.kge_last_error() == b""
    assert loaded.kge_rank_workspace_bytes(4096) >= 4096 * 4 + 8192 * 8
    assert loaded.kge_topk_workspace_bytes(8, 1000, 10) >= 8 * 4096 * 8


def test_host_side_argument_validation_without_gpu(lib_path):
    """Validation happens before anything touches the device, so it can be exercised here."""
    from dicee_amd import _lib
    lib = _lib.load()
    rc = lib.kge_scores(None, None, None, 0, None, 4, 16, 100, None, 100, None)
    assert rc == 1 and b"null" in lib.kge_last_error()
    rc = lib.kge_topk(ctypes.c_void_p(256), None, ctypes.c_void_p(256), 0, None, 4, 16, 100, 200, None, None, 0,
                      None, 0, None)
    assert rc == 1 and b"k=200" in lib.kge_last_error()
    rc = lib.kge_scores(ctypes.c_void_p(256), None, ctypes.c_void_p(256), 2, ctypes.c_void_p(256), 4, 136, 100,
                        ctypes.c_void_p(256), 100, None)
    assert rc == 1 and b"16" in lib.kge_last_error()            # int8 rows need d % 16 == 0
    rc = lib.kge_build_query(3, 1, 1, ctypes.c_void_p(256), 0, None, ctypes.c_void_p(256), 0, None, None, 1, None,
                             ctypes.c_void_p(256), 1, 7, 10, 2, ctypes.c_void_p(256), ctypes.c_void_p(256), None)
    assert rc == 1 and b"Keci" in lib.kge_last_error()
    p256 = ctypes.c_void_p(256)
    rc = lib.kge_csr_build(p256, 10, 0, 1, 1, 5, 5, 5, p256, p256, p256, p256, p256, 1 << 20, None)
    assert rc == 1 and b"permutation" in lib.kge_last_error()
    rc = lib.kge_csr_build(p256, 10, 0, 1, 2, 1 << 30, 1 << 20, 1 << 30, p256, p256, p256, p256, p256, 1 << 20, None)
    assert rc == 2 and b"62-bit" in lib.kge_last_error()
    rc = lib.kge_csr_build(p256, -1, 0, 1, 2, 5, 5, 5, p256, p256, p256, p256, p256, 1 << 20, None)
    assert rc == 1
    # DeCaL goes through its own entry point; the gradient entry points validate before touching the device too
    rc = lib.kge_build_query(5, 1, 1, p256, 0, None, p256, 0, None, None, 1, None, p256, 1, 8, 10, 2, p256, p256, None)
    assert rc == 1 and b"kge_build_query_decal" in lib.kge_last_error()
    rc = lib.kge_build_query_decal(0, 1, 1, 1, p256, 0, None, p256, 0, p256, p256, p256, None, p256, 1, 7, 10, 2, p256,
                                   p256, None)
    assert rc == 1 and b"p + q + r + 1" in lib.kge_last_error()
    rc = lib.kge_build_query_backward(1, 0, 0, 0, p256, p256, None, None, None, 1, p256, 4, 7, 10, 2, p256, None, p256,
                                      p256, None, None, None, None)
    assert rc == 1 and b"ComplEx" in lib.kge_last_error()
    rc = lib.kge_bce_multihot_backward(p256, None, p256, 2, 4, 16, 100, None, None, None, 0, 0.0, 1.0, None, p256, None,
                                       p256, p256, 1 << 30, None)
    assert rc == 2 and b"fp32" in lib.kge_last_error()
    need = lib.kge_bce_backward_workspace_bytes(64, 32, 1000)
    assert need >= 2 * 64 * 1000 * 4 and need % 256 == 0
    rc = lib.kge_bce_multihot_backward(p256, None, p256, 0, 64, 32, 1000, None, None, None, 0, 0.0, 1.0, None, p256, None,
                                       p256, p256, need - 1, None)
    assert rc != 0 and b"workspace" in lib.kge_last_error()
    rc = lib.kge_sample_scores(p256, None, p256, 0, None, 4, 16, 100, None, 3, None, None)
    assert rc == 1 and b"null" in lib.kge_last_error()
    # operands must be 16-byte aligned: the second batch of d = 50 rows sliced out of one array of query vectors is not
    off = ctypes.c_void_p(4096 + 3 * 50 * 4)
    rc = lib.kge_rank_filtered(off, None, p256, 0, None, 3, 50, 100, p256, None, None, None, 0, p256, p256, p256, p256,
                               p256, 1 << 20, None)
    assert rc == 1 and b"16-byte aligned" in lib.kge_last_error()
    # the thresholds of many batches, and the rank call that takes a slice of them: null arrays, a short workspace
    rc = lib.kge_rank_thresholds(p256, None, p256, 0, None, 4, 16, 100, p256, None, p256, p256, p256, p256, None)
    assert rc == 1 and b"threshold" in lib.kge_last_error()
    rc = lib.kge_rank_filtered_with_thresholds(p256, p256, 0, None, 4, 16, 100, p256, None, None, None, None, 0, 1, p256,
                                               p256, p256, p256, 1 << 20, None)
    assert rc == 1 and b"threshold" in lib.kge_last_error()
    rc = lib.kge_rank_filtered_with_thresholds(p256, p256, 0, None, 4, 16, 100, p256, p256, None, None, None, 0, 1, p256,
                                               p256, p256, p256, 8, None)
    assert rc != 0 and b"workspace" in lib.kge_last_error()
    assert lib.kge_rank_thresholds(p256, None, p256, 0, None, 0, 16, 100, None, None, None, None, None, None, None) == 0
    # the measurement aids validate as well
    rc = lib.kge_probe_i8_scan(None, None, 8, 64, ctypes.c_double(1.0), None, None, None)
    assert rc == 1 and b"kge_probe_i8_scan" in lib.kge_last_error()
    rc = lib.kge_probe_mfma(0, 0, ctypes.c_double(100.0), None, None, None)
    assert rc == 1 and b"kge_probe_mfma" in lib.kge_last_error()
    assert lib.kge_profile_kernel() == b""


def test_filter_csr_builders():
    from dicee_amd.csr import FilterCSR
    rng = np.random.default_rng(0)
    N, R, n = 50, 4, 400
    triples = np.stack([rng.integers(0, N, n), rng.integers(0, R, n), rng.integers(0, N, n)], axis=1)
    triples = np.concatenate([triples, triples[:50]])              # duplicates
    brute = {}
    for h, r, t in triples:
        brute.setdefault((int(h), int(r)), set()).add(int(t))
    csr = FilterCSR.from_triples(triples, R)
    keys, row_ptr, col = ko.vocab_csr(triples, "er", R)
    np.testing.assert_array_equal(csr.keys_np, keys)
    np.testing.assert_array_equal(csr.row_ptr_np, row_ptr)
    np.testing.assert_array_equal(csr.col_np, col)
    assert csr.num_rows == len(brute) and csr.nnz == sum(len(v) for v in brute.values())
    for (h, r), tails in brute.items():
        np.testing.assert_array_equal(csr.tails(h, r), sorted(tails))
    er = {}
    for h, r, t in triples:
        er.setdefault((int(h), int(r)), []).append(int(t))         # the reference's list-with-duplicates form
    csr2 = FilterCSR.from_er_vocab(er, R)
    np.testing.assert_array_equal(csr2.row_ptr_np, csr.row_ptr_np)
    np.testing.assert_array_equal(csr2.col_np, csr.col_np)
    rows = csr.rows_for_numpy(np.array([[0, 0], [N + 5, 1], [triples[0, 0], triples[0, 1]]]))
    assert rows[1] == -1 and rows[2] >= 0
    with pytest.raises(RuntimeError):                              # device lookup has no host fallback
        csr.to("cpu").rows_for(torch.tensor([[0, 0]]))
    capped = FilterCSR.from_triples(triples, R, max_per_row=2)
    assert np.diff(capped.row_ptr_np).max() <= 2
    assert len(FilterCSR.from_triples(np.empty((0, 3), dtype=np.int64), R).tails(1, 1)) == 0


def test_metrics_and_tie_rules():
    from dicee_amd.evaluator import compute_metrics_from_ranks_simple, create_hits_dict, update_hits, \
        ranks_from_counts
    ranks = [1, 2, 3, 4, 11, 1, 10]
    hits = create_hits_dict()
    for r in ranks:
        update_hits(hits, r)
    m = compute_metrics_from_ranks_simple(ranks, len(ranks), hits)
    want = ko.metrics_from_ranks(ranks)
    assert m == want
    assert m["MRR"] == pytest.approx(sum(1.0 / r for r in ranks) / len(ranks))
    g, e, l = torch.tensor([0, 5]), torch.tensor([4, 0]), torch.tensor([1, 0])
    assert ranks_from_counts(g, e, l, "stable").tolist() == [2, 6]
    assert ranks_from_counts(g, e, l, "optimistic").tolist() == [1, 6]
    assert ranks_from_counts(g, e, l, "pessimistic").tolist() == [5, 6]
    assert ranks_from_counts(g, e, l, "mean").tolist() == [3, 6]


def test_models_mirror_reference_parameters_and_have_no_cpu_fallback():
    from dicee_amd import models
    args = {"model": "Keci", "embedding_dim": 12, "num_entities": 9, "num_relations": 3, "p": 1, "q": 2}
    m, form = models.initialize_model(args)
    assert form == "EntityPrediction"
    assert set(m.state_dict()) == {"entity_embeddings.weight", "relation_embeddings.weight",
                                   "p_coefficients.weight", "q_coefficients.weight"}
    assert m.r == 3 and float(m.q_coefficients.weight.abs().sum()) == 0.0       # reference init: zeros
    ent, rel = m.get_embeddings()
    assert ent.shape == (9, 12) and rel.shape == (3, 12) and not ent.requires_grad
    c = models.CKeci(args)
    assert float(c.p_coefficients.weight.sum()) == 1.0 and not c.q_coefficients.weight.requires_grad
    with pytest.raises(AssertionError):
        models.Keci({**args, "embedding_dim": 13})
    dc = models.DeCaL({**args, "model": "DeCaL", "embedding_dim": 14, "p": 2, "q": 2, "r": 2})
    assert dc.re == 2 and dc.r_coefficients.weight.shape == (1, 2) and float(dc.r_coefficients.weight.abs().sum()) == 0
    assert set(dc.state_dict()) == {"entity_embeddings.weight", "relation_embeddings.weight", "p_coefficients.weight",
                                    "q_coefficients.weight", "r_coefficients.weight"}
    with pytest.raises(AssertionError):
        models.DeCaL({**args, "model": "DeCaL", "embedding_dim": 15, "p": 2, "q": 2, "r": 2})
    with pytest.raises(ValueError):
        models.initialize_model({**args, "model": "TransE"})
    ln = models.ComplEx({"model": "ComplEx", "embedding_dim": 8, "num_entities": 5, "num_relations": 2,
                         "normalization": "LayerNorm"})
    assert "normalize_head_entity_embeddings.weight" in ln.state_dict()
    d = models.DistMult({"model": "DistMult", "embedding_dim": 8, "num_entities": 5, "num_relations": 2})
    with pytest.raises(RuntimeError):
        d(torch.zeros((2, 2), dtype=torch.int64))                  # CPU tensors: refuses, never falls back
    with pytest.raises(RuntimeError):
        d(torch.zeros((2, 3), dtype=torch.int64))                  # forward_triples: the same rule
    with pytest.raises(RuntimeError):
        d((torch.zeros((2, 2), dtype=torch.int64), torch.zeros((2, 3), dtype=torch.int64)))   # forward_k_vs_sample too
    with pytest.raises(NotImplementedError):
        d(torch.zeros((2, 3, 4), dtype=torch.int64))               # byte-pair-encoded input
    # dropout: in training mode the masks of one forward are drawn from input_dropout_rate (base_model.py:149-151 builds
    # all three modules of this path with it); eval mode and a rate of zero draw none
    dp = models.DistMult({"model": "DistMult", "embedding_dim": 8, "num_entities": 5, "num_relations": 2,
                          "input_dropout_rate": 0.3})
    assert dp.training
    torch.manual_seed(0)
    drop = dp._draw_dropout(1000, "cpu")
    assert set(drop) == {"keep_h", "keep_r", "keep_q", "scale_in", "scale_hidden"}
    assert drop["scale_in"] == pytest.approx(1 / 0.7) and drop["scale_hidden"] == pytest.approx(1 / 0.7)
    for k in ("keep_h", "keep_r", "keep_q"):
        assert drop[k].dtype == torch.uint8 and tuple(drop[k].shape) == (1000, 8)
        assert abs(float(drop[k].float().mean()) - 0.7) < 0.03
    assert set(dp._draw_dropout(4, "cpu", rows=False)) == {"keep_q", "scale_in", "scale_hidden"}
    with pytest.raises(RuntimeError):                              # CPU tensors: refuses, never falls back
        dp(torch.zeros((2, 2), dtype=torch.int64))
    dp.eval()
    assert dp._draw_dropout(4, "cpu") is None
    cx = models.ComplEx({"model": "ComplEx", "embedding_dim": 8, "num_entities": 5, "num_relations": 2,
                         "input_dropout_rate": 0.5})
    assert set(cx._draw_dropout(4, "cpu")) == {"keep_h", "keep_r", "scale_in", "scale_hidden"}
    assert cx._draw_dropout(4, "cpu", rows=False) is None          # only DistMult drops elements of h * r (real.py:32)
    hd = models.ComplEx({"model": "ComplEx", "embedding_dim": 8, "num_entities": 5, "num_relations": 2,
                         "hidden_dropout_rate": 0.1})
    assert hd._draw_dropout(4, "cpu") is None                      # no module of this path is built with that rate


def test_quantised_copies_follow_the_parameters_except_through_weight_data():
    """The bf16 / int8 copies are retaken when the parameters' version or storage changes; an in-place write through
    ``weight.data`` leaves no trace (torch does not advance the version counter), which ``refresh_storage()`` covers."""
    import torch
    from dicee_amd import models
    m = models.DistMult({"embedding_dim": 8, "num_entities": 12, "num_relations": 3})
    m.set_entity_storage("bf16")
    t0 = m.table()[0].clone()
    with torch.no_grad():
        m.entity_embeddings.weight.mul_(2.0)                 # an ordinary in-place update: seen
    assert torch.equal(m.table()[0].float(), t0.float() * 2.0)
    m.entity_embeddings.weight.data.mul_(0.5)                # through .data: not seen ...
    assert torch.equal(m.table()[0].float(), t0.float() * 2.0)
    m.refresh_storage()                                      # ... until asked
    assert torch.equal(m.table()[0].float(), t0.float())
    m.set_entity_storage("int8")
    q0 = m.table()[1].clone()
    m.entity_embeddings.weight.data.mul_(4.0)
    assert torch.equal(m.refresh_storage().table()[1], q0 * 4.0)


def test_evaluating_a_model_on_the_cpu_raises_what_the_ops_raise():
    """There is no CPU path: an evaluation of a model that was never moved to the GPU fails with the ops' own error
    (not with one about streams from the evaluator's batch pipelining)."""
    from types import SimpleNamespace
    from dicee_amd import Evaluator, models
    from dicee_amd.link_prediction import evaluate_lp
    m = models.DistMult({"model": "DistMult", "embedding_dim": 32, "num_entities": 50, "num_relations": 5})
    tr = np.stack([np.arange(20) % 50, np.arange(20) % 5, (np.arange(20) * 7) % 50], 1)
    ev = Evaluator(SimpleNamespace(batch_size=16, eval_model="test", scoring_technique="KvsAll", full_storage_path=None))
    with pytest.raises(RuntimeError, match="GPU"):
        ev.evaluate_lp_k_vs_all(m, tr, form_of_labelling="EntityPrediction")
    er = {(int(h), int(r)): [int(t)] for h, r, t in tr}
    re_ = {(int(r), int(t)): [int(h)] for h, r, t in tr}
    with pytest.raises(RuntimeError, match="GPU"):
        evaluate_lp(m, tr, 50, er, re_, info=None, batch_size=16)


def test_synthetic_configs_small_scale():
    from dicee_amd import synthetic
    c1 = synthetic.make_config("c1")
    assert c1.E.shape == (135, 32) and c1.Rel.shape == (46, 32) and c1.triples.shape == (5216, 3)
    assert c1.queries.shape == (512, 3) and c1.csr.nnz <= 5216
    c4 = synthetic.make_config("c4", scale=0.002)
    assert c4.E.shape[1] == 128 and c4.queries[:, 2].max() < c4.N
    assert np.diff(c4.csr.row_ptr_np).max() <= 50000
    c3 = synthetic.make_config("c3", scale=0.05)
    assert np.diff(c3.csr.row_ptr_np).max() <= 400
    assert len(np.unique(c3.queries[:, 0] * c3.R + c3.queries[:, 1])) == len(c3.queries)
    c5 = synthetic.make_config("c5", scale=0.0001)
    assert c5.csr is None and c5.queries.shape[1] == 3
    p = synthetic.zipf_probs(10, 1.1)
    assert p[0] > p[1] > p[-1] and p.sum() == pytest.approx(1.0)


def test_experiment_folder_round_trip_on_cpu(tmp_path):
    from dicee_amd import models
    from dicee_amd.loader import load_model, save_experiment
    m = models.QMult({"model": "QMult", "embedding_dim": 8, "num_entities": 6, "num_relations": 3})
    ents = {"a,b": 0, "c": 1, "d e": 2, "f": 3, "g": 4, "h": 5}          # names with comma / space survive the csv
    rels = {"r0": 0, "r1": 1, "r2": 2}
    save_experiment(str(tmp_path), m, ents, rels)
    loaded, (e2i, r2i) = load_model(str(tmp_path))
    assert e2i == ents and r2i == rels and loaded.name == "QMult"
    assert all(not p.requires_grad for p in loaded.parameters()) and not loaded.training
    for k, v in m.state_dict().items():
        assert torch.equal(loaded.state_dict()[k], v)
    with pytest.raises(AssertionError):
        load_model(str(tmp_path / "missing"))


def test_three_part_bf16_split_arithmetic():
    """The arithmetic ksplit_kernel relies on, emulated in numpy: an fp32 value is the exact sum of three bf16
    parts (round to nearest even, each part taken from what the previous ones left), and the six leading part
    products summed in fp32 reproduce an fp32 dot product to a few units of 2^-24 of sum(|x||y|)."""
    def bf16_rne(x):
        u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
        u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
        return u.astype(np.uint32).view(np.float32)

    def split3(x):
        parts, r = [], x.astype(np.float32)
        for _ in range(3):
            b = bf16_rne(r)
            parts.append(b)
            r = (r - b).astype(np.float32)
        return parts, r

    rng = np.random.default_rng(7)
    x = (rng.standard_normal(4096) * np.exp(rng.uniform(-8, 8, 4096))).astype(np.float32)
    parts, rest = split3(x)
    assert np.all(rest == 0)                                                 # 3 x 8 significant bits cover fp32's 24
    assert np.array_equal((parts[0].astype(np.float64) + parts[1] + parts[2]).astype(np.float32), x)
    d, n = 256, 64
    X = rng.standard_normal((n, d)).astype(np.float32)
    Y = rng.standard_normal((n, d)).astype(np.float32)
    px, _ = split3(X)
    py, _ = split3(Y)
    order = [(0, 0), (0, 1), (1, 0), (0, 2), (1, 1), (2, 0)]                 # SPLIT_A / SPLIT_B of the kernels
    acc = np.zeros(n, np.float32)
    for k0 in range(0, d, 16):                                               # K steps of 16, fp32 accumulation
        for a, b in order:
            acc = (acc + np.einsum("nk,nk->n", px[a][:, k0:k0 + 16].astype(np.float64),
                                   py[b][:, k0:k0 + 16].astype(np.float64)).astype(np.float32)).astype(np.float32)
    exact = np.einsum("nk,nk->n", X.astype(np.float64), Y.astype(np.float64))
    scale = np.einsum("nk,nk->n", np.abs(X).astype(np.float64), np.abs(Y).astype(np.float64))
    assert np.max(np.abs(acc - exact) / scale) < 2.0 ** -21
    dropped = sum(np.einsum("nk,nk->n", px[a].astype(np.float64), py[b].astype(np.float64))
                  for a, b in [(1, 2), (2, 1), (2, 2)])
    assert np.max(np.abs(dropped) / scale) < 2.0 ** -24


def test_host_logic_builds_and_runs_under_address_and_ub_sanitizers(tmp_path):
    """The library's host logic (csrc/kge_host.h: argument rules, workspace layouts, vocabulary keys, the packed
    counters and the sequential model of the filter-correction plan) compiled by g++ with
    -fsanitize=address,undefined and run on the cases that stress the packed fields: a full sub-batch in one group,
    8192 singleton groups, a 50,000-entry row, a total length at the bound of the work list, int32-long rows."""
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = tmp_path / "host_model_test"
    src = os.path.join(ROOT, "tests", "host_model_test.cpp")
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=all", "-Wall", "-Wextra", "-Werror", "-o", str(exe), src],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    assert "host logic ok" in run.stdout
