#!/usr/bin/env python3
"""Benchmark of the KvsAll filtered-rank / top-k / BCE path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c4] [--no-cpu-baseline]

A step is one pass of the hot path over one batch of synthetic queries: gather + interaction
(kge_build_query), then the fused epilogue the configuration names (filtered rank for c1/c2/c4, BCE for
c3, top-k for c5).  Default workload: c4 = QMult filtered-rank evaluation, 2.5M entities x d=128, bf16
tables with fp32 accumulation, batches of 4096 out of 50k queries whose (h, r) filter rows hold up to
50k known tails.  Tables and index arrays are resident in HBM before the timed region.

Prints ONE JSON line.  `value` = entity scores per second (B*N per step) over the timed region;
`roofline` prices the MFMA main loop (2*d flop per score) against the published dense peak with the
kernel time measured by HIP events on its own stream; `cpu_baseline` times the reference's op sequence
(torch CPU mm + per-row mask loop + full sort) on a small sample of the same queries.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "dice-embeddings_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# MI355X dense bf16 MFMA peak.  fp32 tables run on the same unit: each operand is split into three bf16
# parts and a product is the sum of six bf16 products, so the ceiling for the 2*d flop of an fp32 score is a
# sixth of the bf16 peak (above the 157.3 TFLOP/s of the fp32 MFMA itself).
# int8 tables with d = 128 are scanned for top-k by an int8 x int8 -> int32 MFMA filter (dense int8 peak 5.0 POP/s);
# the candidates it lets through are scored again exactly (int8 row widened to bf16, bf16 x bf16 -> f32).
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 2500.0 / 6.0, "int8": 5000.0}
FP32_MFMA_PEAK_TFLOPS = 157.3
# HBM bytes per launch of the main loop measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on the full-size
# workload (each scaled by what the same counter reads for a plain 1 GiB copy kernel: x2.00 and x1.00).
MEASURED_TRAFFIC_BYTES = {"c4": 660.0e6,     # per rank launch (659 MB read, 1.2 MB written)
                          "c5": 350.0e6,     # average over the 4 filter scans of a top-k call (4.2 GB per call over all kernels)
                          "c3": 59.4e6, "c2": 19.4e6}
MODE = {"c1": "rank", "c2": "rank", "c3": "bce", "c4": "rank", "c5": "topk"}


def cpu_baseline(cfg, model, mode, seconds_budget=25.0):
    """The reference's CPU op sequence (oracle/torch_cpu_path.py) on a bounded sample of the workload."""
    import numpy as np
    import torch
    from oracle import torch_cpu_path as tcp
    threads = torch.get_num_threads()
    E, scale = model.table()
    E = E.float().cpu()
    if scale is not None:
        E = E * scale.float().cpu()[:, None]                    # the dequantised fp32 table
    Rel = model._rel().float().cpu()
    N = E.shape[0]
    name = "Keci" if cfg.model == "Keci" else cfg.model
    kw = {}
    if name == "Keci":
        kw = {"p": cfg.p, "q": cfg.q, "coeff_p": torch.ones(cfg.p), "coeff_q": torch.ones(cfg.q)}
    # sample size: keep B*N*4 bytes of scores around 0.5 GB per batch
    bs = int(max(1, min(cfg.B, (1 << 27) // max(N, 1))))
    q = cfg.queries
    # protocol: one warm-up batch, then timed batches (at least 5 if the budget allows) and the MEDIAN batch time
    # (a workload with fewer batches than that takes them again in turn)
    times = []
    done = 0
    t_spent = 0.0
    n_batches = max(1, len(q) // bs)
    while len(times) < 9 and (len(times) < 5 or t_spent < seconds_budget):
        b_at = (done // bs) % n_batches * bs
        batch = q[b_at:b_at + bs]
        t0 = time.perf_counter()
        if mode == "rank":
            er = {}
            if cfg.csr is not None:
                for h, r, _ in batch:
                    er[(int(h), int(r))] = cfg.csr.tails(int(h), int(r)).astype(np.int64)
            tcp.evaluate_entity_prediction(name, E, Rel, batch, er, bs, **kw)
        elif mode == "topk":
            tcp.predict_topk_indices(name, E, Rel, torch.from_numpy(batch[:, :2].copy()), cfg.k, bs, **kw)
        elif mode in ("bcegrad", "train"):                     # the step with autograd, as loss_batch.backward()
            pos = [cfg.csr.tails(int(h), int(r)).astype(np.int64) for h, r, _ in batch]
            Eg, Rg = E.clone().requires_grad_(), Rel.clone().requires_grad_()
            tcp.kvsall_bce_step(name, Eg, Rg, torch.from_numpy(batch[:, :2].copy()), pos, 0.0, **kw).backward()
        else:
            pos = [cfg.csr.tails(int(h), int(r)).astype(np.int64) for h, r, _ in batch]
            tcp.kvsall_bce_step(name, E, Rel, torch.from_numpy(batch[:, :2].copy()), pos, 0.0, **kw)
        dt = time.perf_counter() - t0
        t_spent += dt
        if done > 0:                                            # the first batch is the warm-up
            times.append(dt)
        done += bs
        if t_spent > 3.0 * seconds_budget:
            break
    if not times:                                               # the budget ran out inside the warm-up batch
        times = [t_spent]
    med = float(np.median(times))
    cpu_model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": bs * N / med, "unit": "scores/s", "cores": threads, "kind": "port",
            "queries_per_sec": bs / med,
            "sample": f"median of {len(times)} timed batches of {bs} queries of {cfg.name} (after one warm-up batch) "
                      f"against all {N} entities, torch {torch.__version__} CPU, {threads} threads, {cpu_model}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c4", choices=sorted(MODE))
    ap.add_argument("--mode", default=None, choices=["rank", "topk", "bce", "bcegrad", "train", "headrank"],
                    help="epilogue to run instead of the configuration's own (headrank: rank the true head of "
                         "(?, r, t) with the (r, t) -> heads filter; bcegrad: BCE loss and its gradients dQ, dbias, dE; "
                         "train: loss and the gradient of every parameter, i.e. bcegrad plus the query builder's backward)")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the workload (testing only)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--streams", type=int, default=1,
                    help="consecutive steps on this many alternating streams, as dicee_amd.Evaluator runs the batches "
                         "of an evaluation (2 there); a step short enough to be a chain of dependent launches gains "
                         "(c2: 0.117 -> 0.075 ms), and the main-loop kernel's own duration then includes what it "
                         "shares the GPU with")
    ap.add_argument("--graph", action="store_true",
                    help="capture one HIP graph per batch before the timed region and replay the graphs (rank, bce and "
                         "bcegrad steps only: the top-k call reads a counter back on the host and cannot be captured)")
    ap.add_argument("--sustain-seconds", type=float, default=2.0,
                    help="length of the `sustained` side run (the same step repeated for this long, after the timed "
                         "region; 0 switches it off)")
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip the `ceiling` side figures (vendor bf16 GEMM on random and on zero operands)")
    ap.add_argument("--no-evaluation-pass", action="store_true",
                    help="skip the `evaluation_pass` side figure (a profile of the step's own launches: the pass runs "
                         "its batches on two streams, where a traced kernel's duration includes its wait for the other's CUs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB-in / 1 GiB-out elementwise kernel (reference point for "
                         "FETCH_SIZE / WRITE_SIZE counters under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no sharding, no collectives); rerun with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from dicee_amd import synthetic, ops

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    mode = args.mode or MODE[args.config]
    t_setup = time.perf_counter()
    big = args.config in ("c4", "c5") and args.scale == 1.0
    cfg = synthetic.make_config(args.config, scale=args.scale, with_tables=not big)
    model = synthetic.make_model(cfg, dev, tables_on_device=big)
    if mode in ("rank", "bce", "bcegrad", "train", "headrank") and cfg.csr is None:
        print(f"bench.py: --mode {mode} needs a configuration with triples", file=sys.stderr)
        sys.exit(2)
    if cfg.csr is not None:
        cfg.csr.to(dev)
    q_all = torch.from_numpy(np.ascontiguousarray(cfg.queries)).to(dev)
    re_csr = None
    if mode == "headrank":
        from dicee_amd.csr import FilterCSR
        re_csr = FilterCSR.from_triples_gpu(torch.from_numpy(np.ascontiguousarray(cfg.triples)).to(dev), cfg.N, cfg.R,
                                            kind="re")
        batches = [(q_all[i:i + cfg.B, 1:].contiguous(), q_all[i:i + cfg.B, 0].contiguous())
                   for i in range(0, len(q_all), cfg.B)]
    else:
        batches = [(q_all[i:i + cfg.B, :2].contiguous(), q_all[i:i + cfg.B, 2].contiguous())
                   for i in range(0, len(q_all), cfg.B)]
    steps = args.steps if args.steps is not None else max(10 * len(batches), 100)
    torch.cuda.synchronize()
    t_setup = time.perf_counter() - t_setup

    def step(i):
        x, t = batches[i % len(batches)]
        if mode == "rank":
            return model.rank_filtered(x, t, cfg.csr)
        if mode == "headrank":
            return model.rank_filtered(x, t, re_csr, heads=True)
        if mode == "topk":
            return model.topk(x, cfg.k)
        if mode == "bcegrad":
            return model.kvsall_bce_backward(x, cfg.csr)
        if mode == "train":
            return model.kvsall_bce_gradients(x, cfg.csr)
        return model.kvsall_bce_loss(x, cfg.csr)

    if args.copy_calibration:
        src = torch.zeros(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)          # reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        del src, dst
    graphs = None
    if args.graph:
        if mode == "topk":
            print("bench.py: --graph does not apply to --mode topk", file=sys.stderr)
            sys.exit(2)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(len(batches)):
                step(i)
        torch.cuda.current_stream().wait_stream(side)
        graphs, keep = [], []
        for i in range(len(batches)):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                keep.append(step(i))
            graphs.append(g)

        def step(i):                                             # noqa: F811 (replaces the eager step on purpose)
            graphs[i % len(graphs)].replay()
    if args.streams > 1:
        if args.graph:
            print("bench.py: --streams does not apply to --graph", file=sys.stderr)
            sys.exit(2)
        pool = [torch.cuda.Stream() for _ in range(args.streams)]
        for s_ in pool:
            s_.wait_stream(torch.cuda.current_stream())
        one_stream_step = step

        def step(i):                                             # noqa: F811 (the same step on alternating streams)
            with torch.cuda.stream(pool[i % len(pool)]):
                return one_stream_step(i)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    ops.profile_begin()
    t0 = time.perf_counter()
    n_queries = 0
    for i in range(steps):
        step(i)
        n_queries += batches[i % len(batches)][0].shape[0]
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_ms, launches = ops.profile_end()
    kernel_name = ops.profile_kernel()                           # what the library dispatched, in its own words

    N, d = cfg.N, cfg.d
    scores = float(n_queries) * N
    compute = "fp32" if cfg.storage == "fp32" else "bf16"
    if cfg.storage == "int8" and mode == "topk" and d == 128:
        compute = "int8"
    flops = 2.0 * d * scores                                    # algorithmic: 2*d flop per entity score
    if mode in ("bcegrad", "train"):
        flops *= 3.0                                            # scores, dQ = g E, dE = g^T Q
    # (inside a replayed graph the launches cannot be bracketed by host-recorded events: no kernel figure then)
    achieved = flops / (kernel_ms * 1e-3) / 1e12 if kernel_ms > 0 else None
    out = {
        "metric": {"rank": "filtered_rank_entity_scores_per_sec", "topk": "topk_entity_scores_per_sec",
                   "bce": "kvsall_bce_entity_scores_per_sec",
                   "bcegrad": "kvsall_bce_forward_backward_entity_scores_per_sec",
                   "train": "kvsall_bce_all_parameter_gradients_entity_scores_per_sec", "headrank": "filtered_head_rank_entity_scores_per_sec"}[mode],
        "value": scores / elapsed,
        "unit": "scores/s",
        "queries_per_sec": n_queries / elapsed,
        "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": elapsed * 1e3 / steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"fp32": "f32 as 3 x bf16 parts, bf16 x bf16 -> f32", "bf16": "bf16 x bf16 -> f32", "int8": "int8 table as bf16 x bf16 -> f32"}[cfg.storage]
                 if compute != "int8" else "int8 x int8 -> i32 filter scan, candidates rescored as bf16 x bf16 -> f32",
        "data": "synthetic",
        "launch": "one HIP graph replay per step" if args.graph else "eager launches" if args.streams <= 1
                  else f"eager launches, consecutive steps alternating over {args.streams} streams",
        "config": {"workload": f"{args.config}: {cfg.model} {mode}, N={N} entities, d={d}, {cfg.storage} tables, "
                               f"batch {cfg.B}, {len(q_all)} queries"
                               + (f", filter CSR nnz={cfg.csr.nnz} max row {int(np.diff(cfg.csr.row_ptr_np).max())}"
                                  if cfg.csr is not None and mode == "rank" else "")
                               + (f", (r,t)->heads CSR nnz={re_csr.nnz} max row {int(np.diff(re_csr.row_ptr_np).max())}"
                                  if mode == "headrank" else "")
                               + (f", k={cfg.k}" if mode == "topk" else ""),
                   "scale": args.scale},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS[compute], "unit": "TFLOP/s",
                     "frac": achieved / PEAK_TFLOPS[compute] if achieved is not None else None,
                     **({"peak_basis": "bf16 dense MFMA 2500 / 6 products per fp32 product",
                         "vs_fp32_mfma_peak": achieved / FP32_MFMA_PEAK_TFLOPS if achieved is not None else None}
                        if compute == "fp32" else
                        {"peak_basis": "int8 dense MFMA, 5.0 POP/s (integer operations, not flop)",
                         "vs_bf16_mfma_peak": achieved / PEAK_TFLOPS["bf16"] if achieved is not None else None}
                        if compute == "int8" else {}),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.config) if mode == MODE[args.config] else None
                     if args.scale == 1.0 and args.mode is None else None,
                     "traffic_source": "measured offline, not in this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on "
                                       "this workload, scaled by a 1 GiB copy kernel (profiles/*_counters.md)",
                     "kernel": kernel_name,
                     "kernel_ms_avg": kernel_ms / max(launches, 1), "launches": launches,
                     "kernel_time_share": kernel_ms * 1e-3 / elapsed},
        "setup_s": t_setup,
        "device": torch.cuda.get_device_name(0),
    }
    # side figure, outside the timed region: the same step repeated for --sustain-seconds, so that the clock the
    # chip settles at under its power limit is inside the figure (the timed region above can be as short as 50 ms)
    if args.sustain_seconds > 0 and not args.graph:
        per_step = elapsed / steps
        n_sus = max(steps, int(args.sustain_seconds / max(per_step, 1e-6)))
        torch.cuda.synchronize()
        ops.profile_begin()
        ts = time.perf_counter()
        nq = 0
        for i in range(n_sus):
            step(i)
            nq += batches[i % len(batches)][0].shape[0]
        torch.cuda.synchronize()
        ts = time.perf_counter() - ts
        k_ms, k_n = ops.profile_end()
        f_sus = 2.0 * d * float(nq) * N * (3.0 if mode in ("bcegrad", "train") else 1.0)
        a_sus = f_sus / (k_ms * 1e-3) / 1e12 if k_ms > 0 else None
        out["sustained"] = {"seconds": ts, "steps": n_sus, "ms_per_step": ts * 1e3 / n_sus,
                            "value": float(nq) * N / ts, "unit": "scores/s",
                            "roofline_achieved": a_sus, "roofline_frac": a_sus / PEAK_TFLOPS[compute] if a_sus else None,
                            "kernel_ms_avg": k_ms / max(k_n, 1), "launches": k_n}
    # side figure, outside the timed region: one whole evaluation pass over every query of the configuration as
    # dicee_amd.Evaluator runs it (vectors, filter rows and thresholds of a group of batches from one launch each,
    # batches alternating over two streams, the ranks formed at the end), wall clock of the best of four passes; and
    # the same pass with every batch on the caller's stream
    if mode in ("rank", "headrank") and not args.graph and not args.no_evaluation_pass:
        from dicee_amd.evaluator import rank_in_batches
        xq = (q_all[:, 1:] if mode == "headrank" else q_all[:, :2]).contiguous()
        tq = (q_all[:, 0] if mode == "headrank" else q_all[:, 2]).contiguous()
        f_csr = re_csr if mode == "headrank" else cfg.csr
        best = {}
        # (streams, call_queries): the evaluator's default merges whole batches into calls of at least 8192 queries
        # (a query's counters do not depend on what else is in its call); 0 keeps one call per batch
        for key in ((2, 8192), (2, 0), (1, 0)):
            for _ in range(4):
                torch.cuda.synchronize()
                tp = time.perf_counter()
                ranks_all = rank_in_batches(model, xq, tq, f_csr, cfg.B, streams=key[0], heads=(mode == "headrank"),
                                            call_queries=key[1])
                torch.cuda.synchronize()
                tp = time.perf_counter() - tp
                best[key] = tp if key not in best else min(best[key], tp)
        n_batches = (int(xq.shape[0]) + cfg.B - 1) // cfg.B
        t_def, t_pb, t_pb1 = best[(2, 8192)], best[(2, 0)], best[(1, 0)]
        out["evaluation_pass"] = {"queries": int(xq.shape[0]), "batch": cfg.B, "streams": 2, "call_queries": 8192,
                                  "ms": t_def * 1e3, "queries_per_sec": xq.shape[0] / t_def,
                                  "value": float(xq.shape[0]) * N / t_def, "unit": "scores/s",
                                  "mrr": float((1.0 / ranks_all.double()).mean().item()),
                                  "one_call_per_batch": {"batches": n_batches, "ms": t_pb * 1e3,
                                                         "ms_per_batch": t_pb * 1e3 / n_batches,
                                                         "one_stream_ms": t_pb1 * 1e3,
                                                         "one_stream_ms_per_batch": t_pb1 * 1e3 / n_batches}}
        del ranks_all
    # side figures, outside the timed region: what the vendor's bf16 GEMM (torch.matmul -> hipBLASLt) sustains on this
    # box, on random and on all-zero operands (the gap is the power limit: random data toggles more), and at the
    # workload's own shape, where it has to write the B x N score matrix that the fused kernels never form
    if not args.no_ceiling and compute in ("bf16", "int8") and args.scale == 1.0:
        def gemm_rate(a_, b_, out_, seconds=0.7):
            for _ in range(3):
                torch.matmul(a_, b_, out=out_)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0_, n_ = time.perf_counter(), 0
            e0.record()
            while True:
                for _ in range(5):
                    torch.matmul(a_, b_, out=out_)
                n_ += 5
                torch.cuda.synchronize()
                if time.perf_counter() - t0_ > seconds:
                    break
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / n_
            return 2.0 * a_.shape[0] * a_.shape[1] * b_.shape[1] / (ms * 1e-3) / 1e12, ms
        ceil = {"unit": "TFLOP/s", "peak": PEAK_TFLOPS["bf16"]}
        g = torch.Generator(device=dev)
        g.manual_seed(1234)
        n_sq = 8192
        A = torch.randn((n_sq, n_sq), device=dev, generator=g).to(torch.bfloat16)
        Bm = torch.randn((n_sq, n_sq), device=dev, generator=g).to(torch.bfloat16)
        C = torch.empty((n_sq, n_sq), device=dev, dtype=torch.bfloat16)
        r, ms = gemm_rate(A, Bm, C)
        ceil["torch_matmul_bf16_8192_cubed_randn"] = {"achieved": r, "frac": r / PEAK_TFLOPS["bf16"], "ms": ms}
        A.zero_()
        Bm.zero_()
        r, ms = gemm_rate(A, Bm, C)
        ceil["torch_matmul_bf16_8192_cubed_zeros"] = {"achieved": r, "frac": r / PEAK_TFLOPS["bf16"], "ms": ms}
        del A, Bm, C
        if compute == "int8":
            # the vendor's int8 GEMM on random int8 operands (int8 x int8 -> int32), against the int8 MFMA peak
            try:
                Ai = torch.randint(-127, 128, (n_sq, n_sq), device=dev, dtype=torch.int8, generator=g)
                Bi = torch.randint(-127, 128, (n_sq, n_sq), device=dev, dtype=torch.int8, generator=g)
                for _ in range(3):
                    torch._int_mm(Ai, Bi)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(20):
                    torch._int_mm(Ai, Bi)
                e1.record()
                torch.cuda.synchronize()
                ms = e0.elapsed_time(e1) / 20
                r = 2.0 * n_sq ** 3 / (ms * 1e-3) / 1e12
                ceil["torch_int_mm_int8_8192_cubed_randint"] = {"achieved": r, "frac": r / PEAK_TFLOPS["int8"], "ms": ms,
                                                                "peak": PEAK_TFLOPS["int8"]}
                del Ai, Bi
            except Exception as exc:                                    # noqa: BLE001 (a side figure: report, go on)
                ceil["torch_int_mm_int8_8192_cubed_randint"] = {"error": f"{type(exc).__name__}: {exc}"[:200]}
        if compute == "int8" and mode == "topk" and model._topk_prepared is not None and model._topk_prepared[1] is not None:
            # the scan's hot loop alone (library measurement aid kge_probe_i8_scan): the same kernel over the whole
            # prepared table with every threshold at +inf, so that no tile passes the bound and nothing is parked or
            # collected; the rounds of a call run the same loop plus the slow path of the tiles that pass
            try:
                xq = batches[0][0]
                Qp, _ = model.query(xq)
                r, ms = ops.probe_i8_scan(Qp, model._topk_prepared[1], N, 1.0)
                ceil["int8_scan_hot_loop_only"] = {
                    "achieved": r, "frac": r / PEAK_TFLOPS["int8"], "ms": ms, "rows": N, "queries": int(Qp.shape[0]),
                    "note": "one launch over all rows; a call's four filter rounds cover the rows past the first 65,536 "
                            "once, so a call's hot-loop time is about this many ms and the rest of its filter time "
                            "is the slow path of the tiles that pass the bound"}
                del Qp
            except Exception as exc:                                    # noqa: BLE001 (a side figure: report, go on)
                ceil["int8_scan_hot_loop_only"] = {"error": f"{type(exc).__name__}: {exc}"[:200]}
        if d == 128 and mode == "rank" and model.table()[0].dtype == torch.bfloat16:
            # the ladder of the rank main loop, bottom up, each rung sustained for ~0.7 s in this process (library
            # measurement aids kge_probe_mfma / kge_probe_walk): the tile statement's MFMAs on random bf16 operands
            # held in registers; with the rank count between them; with the entity fragments re-read from LDS; the
            # whole walk over this table (global -> LDS stages, barriers) without the count.  The top rung is the
            # timed kernel itself (roofline.achieved).
            E_t, _ = model.table()
            Qw, _ = model.query(batches[0][0])
            lad = {}
            for key, (cnt, rd) in (("mfma_registers_only", (0, 0)), ("mfma_with_count", (1, 0)),
                                   ("mfma_with_lds_reads", (0, 1)), ("mfma_with_count_and_lds_reads", (1, 1))):
                r, ms = ops.probe_mfma(cnt, rd, 0.7)
                lad[key] = {"achieved": r, "frac": r / PEAK_TFLOPS["bf16"], "ms": ms}
            r, ms = ops.probe_walk(Qw, E_t, 0.7)
            lad["walk_without_count"] = {"achieved": r, "frac": r / PEAK_TFLOPS["bf16"], "ms": ms,
                                         "shape": [int(Qw.shape[0]), d, N]}
            ceil["rank_main_loop_ladder"] = lad
            del Qw
        if d == 128:
            E_t, _ = model.table()
            if E_t.dtype == torch.bfloat16:
                Bq = batches[0][0].shape[0]
                Qb = torch.randn((Bq, d), device=dev, generator=g).to(torch.bfloat16)
                S_out = torch.empty((Bq, N), device=dev, dtype=torch.bfloat16)
                r, ms = gemm_rate(Qb, E_t.t(), S_out)
                ceil["torch_matmul_bf16_workload_shape"] = {
                    "achieved": r, "frac": r / PEAK_TFLOPS["bf16"], "ms": ms, "shape": [Bq, d, N],
                    "note": "writes the B x N score matrix (bf16) that the fused kernel never forms"}
                del Qb, S_out
        out["ceiling"] = ceil
        torch.cuda.empty_cache()
    # side figure, outside the timed region: the gather + interaction kernel alone (HBM-bound, launch-latency sized)
    xg = batches[0][0]
    for _ in range(3):
        model.query(xg, heads=(mode == "headrank"))
    torch.cuda.synchronize()
    tg = time.perf_counter()
    for _ in range(50):
        model.query(xg, heads=(mode == "headrank"))
    torch.cuda.synchronize()
    tg = (time.perf_counter() - tg) / 50
    esz = {"fp32": 4, "bf16": 2, "int8": 1}[cfg.storage]
    gbytes = xg.shape[0] * d * (esz + (2 if cfg.storage == "bf16" else 4)) + 4 * xg.shape[0] * d + 16 * xg.shape[0]
    out["gather"] = {"kernel": "kge_build_query", "us_per_call": tg * 1e6, "bytes": gbytes,
                     "GB/s": gbytes / tg / 1e9, "frac_of_hbm_peak": gbytes / tg / 8e12,
                     "note": "head and relation rows read, query rows written; wall time of back-to-back calls from Python, "
                             "so launch and binding overhead are inside (the kernel alone: see profiles/)"}
    # the same kernel at the size the evaluation loop runs it: the pairs of up to 64 batches in ONE launch
    # (dicee_amd.evaluator.rank_in_batches), timed with events on the launch stream; bytes = the entity row and the
    # query row of every pair (the relation rows, a few dozen distinct ones, stay in cache) + ids + bias
    n_group = min(len(q_all), 64 * cfg.B)
    xg_all = (q_all[:n_group, 1:] if mode == "headrank" else q_all[:n_group, :2]).contiguous()
    for _ in range(3):
        model.query(xg_all, heads=(mode == "headrank"))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 30
    e0.record()
    for _ in range(reps):
        model.query(xg_all, heads=(mode == "headrank"))
    e1.record()
    torch.cuda.synchronize()
    tgg = e0.elapsed_time(e1) * 1e-3 / reps
    gb_all = n_group * (d * esz + 4 * d + 16 + 4)
    out["gather_grouped"] = {"kernel": "kge_build_query", "pairs": n_group, "us_per_call": tgg * 1e6, "bytes": gb_all,
                             "GB/s": gb_all / tgg / 1e9, "frac_of_hbm_peak": gb_all / tgg / 8e12,
                             "note": "all pairs of an evaluation group in one launch, HIP events around 30 back-to-back "
                                     "launches (allocation of the outputs by torch's caching allocator inside; at this "
                                     "size the host's issue time per call is of the order of the kernel's)"}
    # ... and over about a million pairs (the same pairs repeated), where the kernel's own duration dominates
    rep_n = max(1, (1 << 20) // max(n_group, 1))
    xg_big = xg_all.repeat(rep_n, 1).contiguous()
    for _ in range(2):
        model.query(xg_big, heads=(mode == "headrank"))
    e0.record()
    for _ in range(10):
        model.query(xg_big, heads=(mode == "headrank"))
    e1.record()
    torch.cuda.synchronize()
    tgb = e0.elapsed_time(e1) * 1e-3 / 10
    gb_big = xg_big.shape[0] * (d * esz + 4 * d + 16 + 4)
    out["gather_streaming"] = {"kernel": "kge_build_query", "pairs": int(xg_big.shape[0]), "us_per_call": tgb * 1e6,
                               "bytes": gb_big, "GB/s": gb_big / tgb / 1e9, "frac_of_hbm_peak": gb_big / tgb / 8e12}
    del xg_big
    if len(cfg.triples):
        # side figure, outside the timed region: the known-answer vocabulary of all triples as a CSR, built on
        # the GPU (kge_csr_build) from ids already resident in HBM
        from dicee_amd.csr import FilterCSR
        trip = torch.from_numpy(np.ascontiguousarray(cfg.triples)).to(dev)
        FilterCSR.from_triples_gpu(trip, N, cfg.R)                 # warm-up (allocator, code objects)
        torch.cuda.synchronize()
        tb = time.perf_counter()
        built = FilterCSR.from_triples_gpu(trip, N, cfg.R)
        torch.cuda.synchronize()
        tb = time.perf_counter() - tb
        out["csr_build"] = {"ms": tb * 1e3, "triples": int(trip.shape[0]), "rows": built.num_rows, "nnz": built.nnz,
                            "triples_per_sec": trip.shape[0] / tb}
        del trip, built
    if not args.no_cpu_baseline and mode != "headrank":
        out["cpu_baseline"] = cpu_baseline(cfg, model, mode)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
