#!/usr/bin/env python3
"""Benchmark of the MI355X token-sampling path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the sampling path over one batch of synthetic logit rows that already
sit in HBM: penalties + temperature + top-k + top-p + draw for the default workload
(B = 64 x V = 128256 fp32, T = 0.7, top-k 40, top-p 0.9, one seeded uniform per row, history of
2048 Zipf ids per row with repetition 1.1 / frequency 0.5 / presence 0.3). Prints ONE JSON line.

value      rows sampled per second over the timed K steps (whole job, one GPU). The steps rotate
           over copies of the batch that together exceed the caches, so every step streams its
           logits from HBM; `rows_per_s_cache_resident` is the same loop on one buffer, whose
           logits the 256 MB Infinity Cache keeps between steps
roofline   the logit-streaming kernel: algorithmic bytes per launch / its mean duration, the
           duration taken with HIP events on the sampler's stream around K back-to-back launches
           of that kernel alone over the same rotating copies, right after the timed region
cpu_baseline  the CPU restatement of the same step (oracle, reference build flags) timed on
           this host's cores on a bounded sample; reported, not the optimisation target
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
COLD_WORKING_SET = 640 * 1024 * 1024   # bytes of logits the timed loops cycle through

# HBM bytes moved by one launch of the step's kernel, from rocprofv3's FETCH_SIZE and
# WRITE_SIZE scaled by what the same counters read for a plain copy of the logit buffer. A
# counter run cannot happen inside a timed benchmark, so the figure is carried here together
# with the summary it was taken from (`roofline.traffic_source`); workloads without a counter
# run report null.
PROFILED_TRAFFIC = {
    "cfg2_b64_v128256_pen2048": (35264326, "profiles/k_cand_scan_final__cfg2_pen.md"),
    "cfg2_b64_v128256": (34624496, "profiles/k_cand_scan_final__cfg2.md"),
}


def build_workload(name):
    from geistlib_amd import workloads as W
    if name == "cfg2_pen":
        return W.config2(with_penalties=True)
    if name == "cfg2":
        return W.config2(with_penalties=False)
    if name.startswith("cfg2_pen_b") or name.startswith("cfg2_b"):
        # the headline's parameters on another number of rows (cfg2_pen_b1: one decode step of
        # one session, which is what the reference's geist_session_decode_step samples)
        return W.config2(rows=int(name.split("_b")[1]), with_penalties=name.startswith("cfg2_pen"))
    if name == "cfg3":
        return W.config3()
    if name == "cfg4":
        return W.config4()
    if name == "cfg1":
        return W.config1()
    if name == "cfg5":
        return W.config5()
    raise SystemExit(f"unknown workload {name}")


def cpu_baseline(w, budget_s=20.0):
    """Times the oracle (built with the reference's release flags) on this host."""
    from oracle_lib import Oracle
    try:
        o = Oracle(fast=True)
    except Exception as e:  # the oracle objects are test infrastructure; absence is not fatal
        return {"value": None, "unit": "rows/s", "cores": 0, "kind": "port",
                "sample": f"oracle unavailable: {e}"}, None
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 10 ** 6,
                o.lib.oracle_max_threads())
    kw = dict(temperature=w.temperature, top_k=w.top_k, top_p=w.top_p, min_p=w.min_p,
              hist=w.history, hist_len=w.history_len, rep=w.rep, freq=w.freq, pres=w.pres)
    out = {}
    for label, threads in (("1", 1), ("all", cores)):
        o.batch_chain_u(w.logits[:min(4, w.rows)], w.uniforms, threads=threads, **{
            **kw, "hist": None if w.history is None else w.history[:4],
            "hist_len": None if w.history_len is None else w.history_len[:4]})  # warm-up
        reps, t_used = 0, 0.0
        while reps < 10 and t_used < budget_s / 2:
            t0 = time.perf_counter()
            ids = o.batch_chain_u(w.logits, w.uniforms, threads=threads, **kw)
            t_used += time.perf_counter() - t0
            reps += 1
        out[label] = (w.rows * reps / t_used, reps, ids)
    v_all, reps_all, ids = out["all"]
    v_1, reps_1, _ = out["1"]
    return {"value": round(v_all, 2), "unit": "rows/s", "cores": cores, "kind": "port",
            "single_core_rows_per_s": round(v_1, 2),
            **reference_top_k_baseline(w, cores, budget_s / 2),
            "sample": f"whole batch of {w.rows} rows x {reps_all} repeats on {cores} threads "
                      f"(one row per thread) and x {reps_1} repeats on 1 thread; oracle built with "
                      "-O3 -ffast-math -march=x86-64-v3 -fopenmp"}, ids


def reference_top_k_baseline(w, cores, budget_s):
    """Times the reference's own geist_sampler_top_k_ws (src/engine/sampler.c:178-228, compiled
    from its sources with its release flags) on the same rows: k and temperature of the workload,
    reference precedence (top-k alone, no top-p, no penalties). One workspace and one generator
    per thread, as the reference's sessions hold them. Empty where that library was not built."""
    import ctypes as C
    import threading
    from oracle_lib import load_ref, RefWorkspace, OracleRng
    lib = load_ref(fast=True)
    if lib is None or w.top_k <= 0 or w.temperature <= 0:
        return {}
    fp = C.POINTER(C.c_float)
    rows = [np.ascontiguousarray(r, dtype=np.float32) for r in w.logits]

    def work(mine, reps, counter):
        ws, rng = RefWorkspace(), OracleRng()
        if lib.geist_sampler_workspace_init(C.byref(ws), w.n_vocab) != 0:
            return
        lib.geist_rng_seed(C.byref(rng), 1234)
        for _ in range(reps):
            for i in mine:
                lib.geist_sampler_top_k_ws(C.byref(ws), rows[i].ctypes.data_as(fp), w.top_k,
                                           w.temperature, C.byref(rng))
                counter[0] += 1
        lib.geist_sampler_workspace_destroy(C.byref(ws))

    res = {}
    for label, threads in (("1", 1), ("all", cores)):
        # size the sample from one timed row so that each leg takes a few seconds
        c = [0]
        t0 = time.perf_counter()
        work([0], 1, c)
        per_row = max(time.perf_counter() - t0, 1e-6)
        want = budget_s / 2 / per_row * threads
        reps = max(1, min(10, int(want / w.rows)))
        n_rows = w.rows if want >= w.rows else max(threads, int(want))
        shares = [list(range(t, n_rows, threads)) for t in range(threads)]
        counters = [[0] for _ in range(threads)]
        th = [threading.Thread(target=work, args=(shares[t], reps, counters[t]))
              for t in range(threads)]
        t0 = time.perf_counter()
        for t in th:
            t.start()
        for t in th:
            t.join()
        dt = time.perf_counter() - t0
        res[label] = (sum(c[0] for c in counters) / dt, n_rows, reps)
    return {"reference_top_k_rows_per_s": round(res["all"][0], 2),
            "reference_top_k_single_core_rows_per_s": round(res["1"][0], 2),
            "reference_top_k_sample": f"geist_sampler_top_k_ws(k={w.top_k}, T={w.temperature}) from "
                                      f"oracle/_ref (release flags): {res['all'][1]} rows x "
                                      f"{res['all'][2]} on {cores} threads, {res['1'][1]} rows x "
                                      f"{res['1'][2]} on 1 thread"}


def topk_path_counts(hs, row_sets, prm, d_u, d_out, n_rows):
    """Which path served the rows of a top-k configuration, over every input copy once
    (geist_hip_sampler_topk_paths after each call): the candidates handed on by the scan, the
    per-thread maxima, the selection over the whole row; fallback_rate = the share of rows that
    did not take the first."""
    counts = {"scan_candidates": 0, "thread_maxima": 0, "whole_row": 0, "other": 0}
    for rs in row_sets:
        hs.sample(rs, prm, d_u, d_out)
        for p in hs.topk_paths(n_rows).tolist():
            counts[{0: "scan_candidates", 1: "thread_maxima", 2: "whole_row"}.get(p, "other")] += 1
    total = max(1, sum(counts.values()))
    counts["rows"] = total
    counts["fallback_rate"] = round(1.0 - counts["scan_candidates"] / total, 6)
    return counts


def time_other_configs(steps=50, warmup=10):
    """The other four benchmark configurations under the same clock as the headline workload:
    `steps` HBM-cold steps each (the inputs rotate over copies that together exceed the Infinity
    Cache), wall-clock per step, and -- for the configurations that are one sampling call -- the
    logit-streaming kernel on its own by HIP events. Inputs are drawn on the device with the
    configurations' distributions (parity of these configurations at full size is the business of
    tests/test_gpu_configs.py, not of this leg); no CPU leg."""
    import torch
    from geistlib_amd import HipSampler, SampleParams
    from geistlib_amd import bench_hooks as bh
    from geistlib_amd.workloads import zipf_history
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    out = {}

    def normal(shape, scale):
        return torch.randn(shape, device=dev, generator=g) * scale

    def run(name, make_copy, n_copies, rows, n_vocab, prm_kw, hist_len=0, extra_bytes=0,
            fast_sums_twin=False):
        copies = [make_copy() for _ in range(n_copies)]
        d_u = torch.rand(rows, device=dev, generator=g)
        d_out = torch.empty(rows, dtype=torch.int32, device=dev)
        d_h = d_hl = None
        if hist_len:
            hg = np.random.default_rng(3)
            d_h = torch.from_numpy(zipf_history(hg, rows, hist_len, n_vocab)).to(dev)
            d_hl = torch.full((rows,), hist_len, dtype=torch.int32, device=dev)
        hs = HipSampler(max_rows=rows, max_vocab=n_vocab)
        hs.set_logits_hint(True)
        prm = SampleParams.make(**prm_kw)
        hs.prepare(prm, n_vocab)
        rl = [HipSampler.rows(c, d_h, d_hl) for c in copies]
        for i in range(max(warmup, n_copies)):
            hs.sample(rl[i % n_copies], prm, d_u, d_out)
        hs.sync()
        t0 = time.perf_counter()
        for i in range(steps):
            hs.sample(rl[i % n_copies], prm, d_u, d_out)
        hs.sync()
        us = (time.perf_counter() - t0) * 1e6 / steps
        k_us, k_name = bh.time_stream_kernel(hs, rl, prm, d_u, d_out, steps)
        alg = rows * (4 * n_vocab + 8) + extra_bytes
        out[name] = {"us_per_step": round(us, 2), "rows_per_s": round(rows / (us * 1e-6), 1),
                     "step_frac": round(alg / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     "step_algorithmic_bytes": int(alg), "kernel": k_name,
                     "kernel_us": round(k_us, 2), "steps": steps, "input_copies_rotated": n_copies}
        if prm_kw.get("top_k"):
            out[name]["topk_paths"] = topk_path_counts(hs, rl, prm, d_u, d_out, rows)
        if fast_sums_twin:
            # the same with the sums of exponentials from the hardware's 2^z (the contract's
            # tolerance used, geist_hip_sampler_set_sums; off by default)
            hs.set_sums(fast=True)
            for i in range(max(warmup, n_copies)):
                hs.sample(rl[i % n_copies], prm, d_u, d_out)
            hs.sync()
            t0 = time.perf_counter()
            for i in range(steps):
                hs.sample(rl[i % n_copies], prm, d_u, d_out)
            hs.sync()
            out[name]["us_per_step_fast_sums"] = round((time.perf_counter() - t0) * 1e6 / steps, 2)
            out[name]["kernel_us_fast_sums"] = round(
                bh.time_stream_kernel(hs, rl, prm, d_u, d_out, steps)[0], 2)
        hs.close()

    # cfg1: one row of 128256, N(0, 3^2), T = 0.8 (the rows of a [1400 x V] buffer take turns)
    big = normal((1400, 128256), 3.0)
    run("cfg1", iter([big[i:i + 1] for i in range(1400)]).__next__, 1400, 1, 128256,
        dict(temperature=0.8))
    # one decode step of one session, which is what the reference's sample call serves
    # (geist_session_decode_step): one row with the headline's parameters and penalties
    run("decode_one_row", iter([big[i:i + 1] for i in range(1400)]).__next__, 1400, 1, 128256,
        dict(temperature=0.7, top_k=40, top_p=0.9, rep=1.1, freq=0.5, pres=0.3), hist_len=2048,
        extra_bytes=4 * 2048 + 8 * 1000)
    del big
    # cfg3: 128 x 151936, N(0, 2^2), Zipf history of 2048, penalties, T = 1, top-p 0.95, min-p 0.05
    hist_bytes = 128 * (4 * 2048 + 8 * 1000)   # ids read + about 1000 distinct per row gathered
    run("cfg3", lambda: normal((128, 151936), 2.0), 9, 128, 151936,
        dict(temperature=1.0, top_p=0.95, min_p=0.05, rep=1.1, freq=0.5, pres=0.3), hist_len=2048,
        extra_bytes=hist_bytes, fast_sums_twin=True)
    # cfg4: 256 x 262144, Student-t(3) x 2.5, top-k 64 -> top-p 0.9, T = 0.6
    def student_t():
        z = torch.randn((256, 262144), device=dev, generator=g)
        chi = (torch.randn((3, 256, 262144), device=dev, generator=g) ** 2).sum(0)
        return (z / torch.sqrt(chi / 3.0) * 2.5).contiguous()
    run("cfg4", student_t, 3, 256, 262144, dict(temperature=0.6, top_k=64, top_p=0.9))
    # cfg5: 32 sequences x 9 target rows of 128256, q = softmax(target + N(0, 0.5^2))
    n_seq, L, V = 32, 8, 128256
    ts, qs = [], []
    for _ in range(3):
        t = normal((n_seq, L + 1, V), 2.0)
        q = torch.softmax((t[:, :L, :] + normal((n_seq, L, V), 0.5)).double(), dim=-1).float()
        ts.append(t)
        qs.append(q.contiguous())
    draft = torch.multinomial(qs[0].reshape(-1, V), 1, generator=g).reshape(n_seq, L).to(torch.int32)
    u = torch.rand((n_seq, L + 1), device=dev, generator=g)
    o_tok = torch.full((n_seq, L + 1), -1, dtype=torch.int32, device=dev)
    nacc = torch.full((n_seq,), -1, dtype=torch.int32, device=dev)
    hs = HipSampler(max_rows=n_seq * (L + 1), max_vocab=V)
    hs.set_logits_hint(1)
    for i in range(max(warmup, 3)):
        hs.spec_verify(ts[i % 3], qs[i % 3], draft, u, 1.0, o_tok, nacc)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(steps):
        hs.spec_verify(ts[i % 3], qs[i % 3], draft, u, 1.0, o_tok, nacc)
    hs.sync()
    us = (time.perf_counter() - t0) * 1e6 / steps
    rows = n_seq * (L + 1)
    alg = rows * V * 4 + n_seq * V * 4 + rows * 8 + n_seq * 4
    out["cfg5"] = {"us_per_step": round(us, 2), "rows_per_s": round(rows / (us * 1e-6), 1),
                   "sequences_per_s": round(n_seq / (us * 1e-6), 1),
                   "step_frac": round(alg / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                   "step_algorithmic_bytes": int(alg),
                   "kernel": "k_scan_expsum + k_spec_resid_draw (whole step)", "kernel_us": None,
                   "steps": steps, "input_copies_rotated": 3}
    hs.set_sums(fast=True)
    for i in range(max(warmup, 3)):
        hs.spec_verify(ts[i % 3], qs[i % 3], draft, u, 1.0, o_tok, nacc)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(steps):
        hs.spec_verify(ts[i % 3], qs[i % 3], draft, u, 1.0, o_tok, nacc)
    hs.sync()
    out["cfg5"]["us_per_step_fast_sums"] = round((time.perf_counter() - t0) * 1e6 / steps, 2)
    hs.close()
    return out


def bench_spec(w, args):
    """Configuration 5: speculative verification of n_seq sequences x (L + 1) target rows. A step
    is one geist_hip_spec_verify call; rows/s counts target rows."""
    import torch
    from geistlib_amd import HipSampler
    x = w.extra
    n_seq, L = x["n_seq"], x["draft_len"]
    dev = torch.device("cuda:0")
    # three copies of the inputs (840 MB against the 256 MB Infinity Cache): every step reads its
    # target rows and draft probabilities from HBM
    n_copies = 3
    ts = [torch.from_numpy(x["target"]).to(dev) for _ in range(n_copies)]
    qs = [torch.from_numpy(x["q"]).to(dev) for _ in range(n_copies)]
    d = torch.from_numpy(x["draft"]).to(dev)
    u = torch.from_numpy(x["uniforms"]).to(dev)
    out = torch.full((n_seq, L + 1), -1, dtype=torch.int32, device=dev)
    nacc = torch.full((n_seq,), -1, dtype=torch.int32, device=dev)
    hs = HipSampler(max_rows=n_seq * (L + 1), max_vocab=w.n_vocab)
    hs.set_logits_hint(1)   # the rows come from HBM and are read once
    if args.fast_sums:
        hs.set_sums(fast=True)

    def step(i):
        hs.spec_verify(ts[i % n_copies], qs[i % n_copies], d, u, w.temperature, out, nacc)

    for i in range(max(args.warmup, n_copies)):
        step(i)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    hs.sync()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps
    rows = n_seq * (L + 1)
    # every target logit once, one row of draft probabilities per sequence (the rejected
    # position's), uniforms in, ids and counts out
    alg = rows * w.n_vocab * 4 + n_seq * w.n_vocab * 4 + rows * 4 + rows * 4 + n_seq * 4
    achieved = alg / (ms * 1e-3) / 1e9
    result = {
        "metric": "sampled rows/s", "value": round(rows * args.steps / elapsed, 1),
        "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": w.name, "sums": "fast" if args.fast_sums else "exact",
                   "sequences": n_seq, "draft_len": L, "n_vocab": w.n_vocab,
                   "temperature": w.temperature},
        "us_per_step": round(ms * 1e3, 3),
        "sequences_per_s": round(n_seq * args.steps / elapsed, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "whole step (two kernels)", "step_algorithmic_bytes": alg},
        "input_copies_rotated": n_copies,
        "accepted_lengths": sorted(nacc.cpu().numpy().tolist()),
    }
    if not args.no_cpu:
        result["cpu_baseline"], want = spec_cpu_baseline(w)
        got_n, got_out = nacc.cpu().numpy(), out.cpu().numpy()
        differ = sum(int(got_n[s_] != n_) or got_out[s_, :n_ + 1].tolist() != o_[:n_ + 1].tolist()
                     for s_, (n_, o_) in enumerate(want))
        result["parity"] = {"sequences": n_seq, "verdicts_differ": int(differ)}
    print(json.dumps(result))


def spec_cpu_baseline(w, budget_s=15.0):
    """The oracle's speculative verification (built with the reference's release flags) on this
    host: every sequence of the batch, one sequence per thread; repeated to fill the budget."""
    from concurrent.futures import ThreadPoolExecutor
    from oracle_lib import Oracle
    x = w.extra
    n_seq = x["n_seq"]
    o = Oracle(fast=True)
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 10 ** 6)

    def one(s):
        return o.spec_verify(x["target"][s], x["q"][s], x["draft"][s], x["uniforms"][s],
                             w.temperature)

    with ThreadPoolExecutor(cores) as pool:
        list(pool.map(one, range(min(cores, n_seq))))        # warm-up
        reps, t_used, res = 0, 0.0, None
        while reps < 10 and t_used < budget_s:
            t0 = time.perf_counter()
            res = list(pool.map(one, range(n_seq)))
            t_used += time.perf_counter() - t0
            reps += 1
    rows = n_seq * (x["draft_len"] + 1)
    return {"value": round(rows * reps / t_used, 2), "unit": "rows/s", "cores": cores,
            "kind": "port",
            "sample": f"the whole batch of {n_seq} sequences x {reps} repeats on {cores} threads "
                      "(one sequence per thread); oracle built with -O3 -ffast-math "
                      "-march=x86-64-v3"}, res


def bench_lm_head(args, m_rows, q8=False):
    """Workload lm_head[_q8][_mN]: the tail of a decode step for BitNet-2B-4T's geometry, the case the
    reference's F16 lm_head kernel was written for (cpu_x86/kernel_f16_gemv.h:7-12): RMS norm of
    the hidden row(s), the tied F16 lm_head [128256 x 2560] (657 MB, read once per step), then the
    headline sampler configuration on the logits, which never leave the device. A step is one
    such tail for m_rows rows; the dominant kernel is the projection. With q8 the table is the
    int8 form the reference's x86 backend decodes with (cpu_x86/backend.c:332-372: 328 MB + one
    scale per row), quantised on the device from the same F16 tables."""
    import torch
    from geistlib_amd import HipSampler, SampleParams
    from geistlib_amd.workloads import xorshift_units
    vocab, d_model = 128256, 2560
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    # three copies of the table (1.97 GB): every step's weights come from HBM
    tables = [(torch.randn((vocab, d_model), device=dev, generator=g) * 0.05).to(torch.float16)
              for _ in range(3)]
    hidden = torch.randn((m_rows, d_model), device=dev, generator=g) * 3
    norm_w = 1.0 + 0.1 * torch.randn((d_model,), device=dev, generator=g)
    u, _ = xorshift_units(7, m_rows)
    d_u = torch.from_numpy(u).to(dev)
    normed = torch.empty_like(hidden)
    logits = torch.empty((m_rows, vocab), dtype=torch.float32, device=dev)
    out = torch.empty(m_rows, dtype=torch.int32, device=dev)
    hs = HipSampler(max_rows=max(m_rows, 1), max_vocab=vocab)
    prm = SampleParams.make(temperature=0.7, top_k=40, top_p=0.9)
    if q8:
        tables_q8 = [torch.empty((vocab, d_model), dtype=torch.int8, device=dev) for _ in tables]
        scales = [torch.empty(vocab, dtype=torch.float32, device=dev) for _ in tables]
        for t, tq, sc in zip(tables, tables_q8, scales):
            hs.f16_to_q8w(t, tq, sc)
        hs.sync()

    def step(i=0):
        j = i % len(tables)
        if q8:
            hs.project_sample_q8w(hidden, norm_w, 1e-6, tables_q8[j], scales[j], logits, prm, d_u,
                                  out, normed=normed)
        else:
            hs.project_sample(hidden, norm_w, 1e-6, tables[j], logits, prm, d_u, out,
                              normed=normed)

    for i in range(args.warmup):
        step(i)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    hs.sync()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps
    ids_gpu = out.cpu().numpy()
    hs.rmsnorm(hidden, norm_w, 1e-6, normed)
    # the projection alone
    f64_batch = (not q8) and m_rows > 1   # what project_sample runs for more than one F16 row
    from geistlib_amd.bench_hooks import Timer

    def projection(i):
        j = i % len(tables)
        if q8:
            hs.q8w_gemv(tables_q8[j], scales[j], normed, logits)
        elif not f64_batch:
            hs.f16_gemv(tables[j], normed, logits)
        else:
            hs.f16_linear(tables[j], normed, logits)

    for i in range(len(tables)):
        projection(i)
    with Timer() as tm:       # HIP events on the sampler's stream around the launches
        for i in range(args.steps):
            projection(i)
    kernel_us = tm.ms * 1e3 / args.steps
    w_bytes = vocab * d_model + vocab * 4 if q8 else vocab * d_model * 2
    achieved = w_bytes / (kernel_us * 1e-6) / 1e9
    result = {
        "metric": "sampled rows/s", "value": round(m_rows * args.steps / elapsed, 1),
        "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("int8" if q8 else "f16") + " weights x f32 activations, "
                 + ("f64" if (not q8 and m_rows > 1) else "f32") + " accumulation",
        "data": "synthetic",
        "config": {"workload": f"lm_head{'_q8' if q8 else ''}_v{vocab}_d{d_model}_m{m_rows}",
                   "rows": m_rows,
                   "n_vocab": vocab, "d_model": d_model, "temperature": 0.7, "top_k": 40,
                   "top_p": 0.9},
        "us_per_step": round(ms * 1e3, 3),
        "weight_copies_rotated": len(tables),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": ("k_q8w_gemv" if q8 else
                                "k_f16_linear_f64 (+ activations to double, listed outputs)"
                                if f64_batch else "k_f16_gemv"),
                     "kernel_us": round(kernel_us, 3),
                     "kernel_algorithmic_bytes": w_bytes,
                     "step_algorithmic_bytes": w_bytes + m_rows * (d_model * 8 + vocab * 8 + 8)},
    }
    if f64_batch:
        # a batch is bound by double-precision arithmetic, not by the one pass over the table
        flops = 2.0 * m_rows * vocab * d_model
        tf = flops / (kernel_us * 1e-6) / 1e12
        result["roofline"].update({"bound": "mfma", "achieved": round(tf, 2), "peak": 78.6,
                                   "unit": "TFLOP/s", "frac": round(tf / 78.6, 4),
                                   "kernel_algorithmic_flops": flops})
    if not args.no_cpu:
        # the reference's own kernel, compiled from its tree (oracle/_ref), on this host's cores;
        # where it was not built, the oracle's scalar restatement on one core
        from oracle_lib import Oracle, load_ref_f16gemv
        wt = tables[(args.steps - 1) % len(tables)].cpu().numpy().view(np.uint16)
        x_host = normed.cpu().numpy()
        o = Oracle()
        ref = load_ref_f16gemv(fast=True)
        y = np.empty(vocab, dtype=np.float32)
        if q8:
            wq, sc = o.f16_to_q8w(wt)
        fp = C.POINTER(C.c_float)
        reps, t_used = 0, 0.0
        while f64_batch and reps < 3 and t_used < 10.0:
            # a batch: the portable kernel (the oracle's restatement, rows spread over the cores
            # as nothing in the reference does: its loop is serial)
            t1 = time.perf_counter()
            o.f16_linear_f64(wt, x_host)
            t_used += time.perf_counter() - t1
            reps += 1
        while not f64_batch and reps < 10 and t_used < 10.0:
            t1 = time.perf_counter()
            if ref is not None and q8:
                ref.q8w_gemv_m1(vocab, d_model, x_host[0].ctypes.data_as(fp),
                                wq.ctypes.data_as(C.POINTER(C.c_int8)), sc.ctypes.data_as(fp),
                                y.ctypes.data_as(fp))
            elif ref is not None:
                ref.f16_gemv_m1(vocab, d_model, x_host[0].ctypes.data_as(fp),
                                wt.ctypes.data_as(C.POINTER(C.c_uint16)), y.ctypes.data_as(fp))
            elif q8:
                y = o.q8w_gemv(wq, sc, x_host[0])
            else:
                y = o.f16_gemv(wt, x_host[0])
            t_used += time.perf_counter() - t1
            reps += 1
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 10 ** 6)
        if f64_batch:
            result["cpu_baseline"] = {
                "value": round(reps * m_rows / t_used, 2), "unit": "rows/s", "cores": cores,
                "kind": "port",
                "sample": f"{reps} calls of the double-accumulation projection on the batch of "
                          f"{m_rows} rows (no norm, no sampling)"}
        else:
            result["cpu_baseline"] = {
                "value": round(reps / t_used, 2), "unit": "rows/s",
                "cores": cores if ref is not None else 1,
                "kind": "reference" if ref is not None else "port",
                "sample": f"{reps} calls of {'q8w' if q8 else 'f16'}_gemv_m1 on one hidden row "
                          "(the projection only, no norm, no sampling)"}
        # parity of the whole tail on the last step's inputs
        x_normed = o.rmsnorm(hidden.cpu().numpy(), norm_w.cpu().numpy(), 1e-6)
        want_logits = (o.q8w_gemv(wq, sc, x_normed) if q8 else
                       o.f16_linear_f64(wt, x_normed) if f64_batch else o.f16_gemv(wt, x_normed))
        same_bits = bool((want_logits.view(np.uint32) == logits.cpu().numpy().view(np.uint32)).all())
        want_ids = [o.chain_u(want_logits[r], float(u[r]), temperature=0.7, top_k=40, top_p=0.9)[0]
                    for r in range(m_rows)]
        result["parity"] = {"rows": m_rows, "logits_bit_identical": same_bits,
                            "ids_differ": int((np.array(want_ids) != ids_gpu).sum())}
        if q8:
            j = (args.steps - 1) % len(tables)
            result["parity"]["table_bit_identical"] = bool(
                (tables_q8[j].cpu().numpy() == wq).all()
                and (scales[j].cpu().numpy().view(np.uint32) == sc.view(np.uint32)).all())
    print(json.dumps(result))


class _DevPtr:
    """A device array known by its address only, for the timing entry points."""

    def __init__(self, ptr, shape):
        self.ptr, self.shape = ptr, shape

    def data_ptr(self):
        return self.ptr

    def is_contiguous(self):
        return True

    def element_size(self):
        return 1


def bench_lm_head_q6k(args, m_rows):
    """Workload lm_head_q6k[_mN]: the tail of a decode step for the geometry of the Gemma models,
    whose tied embedding is a Q6_K table (the reference resolves it at
    src/backends/cpu_x86/backend.c:395-397, the portable kernel at
    src/backends/cpu_scalar/weight_resolve.c:86-88, 186-241): RMS norm, the lm_head over
    [262144 x 1536] Q6_K super-blocks (330 MB, read once per step), then soft-cap 30 and the
    headline sampler configuration on logits that never leave the device. The dominant kernel is
    the projection; its algorithmic bytes are the table's."""
    import torch
    from geistlib_amd import HipSampler, SampleParams
    from geistlib_amd.bench_hooks import Timer
    from geistlib_amd.workloads import xorshift_units
    vocab, d_model = 262144, 1536
    nb = d_model // 256
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    tables = []
    for _ in range(3):          # three copies (1 GB): every step's table comes from HBM
        t = torch.randint(0, 256, (vocab, nb, 210), dtype=torch.uint8, device=dev, generator=g)
        # scales 0..15 and d = binary16 0x0C6D = 2.7e-4 in every block: logits of a few units,
        # as a model's are (random scales and d would saturate the soft-cap into one huge tie)
        t[:, :, 192:208] &= 0x0F
        t[:, :, 208] = 0x6D
        t[:, :, 209] = 0x0C
        tables.append(t.reshape(vocab, nb * 210).contiguous())
    hidden = torch.randn((m_rows, d_model), device=dev, generator=g) * 3
    norm_w = 1.0 + 0.1 * torch.randn((d_model,), device=dev, generator=g)
    u, _ = xorshift_units(7, m_rows)
    d_u = torch.from_numpy(u).to(dev)
    normed = torch.empty_like(hidden)
    logits = torch.empty((m_rows, vocab), dtype=torch.float32, device=dev)
    out = torch.empty(m_rows, dtype=torch.int32, device=dev)
    hs = HipSampler(max_rows=max(m_rows, 1), max_vocab=vocab)
    prm = SampleParams.make(temperature=0.7, top_k=40, top_p=0.9, softcap=30.0)

    # the copies of the tables in the order the device reads them (geist_hip_q6k_pack, once per
    # model at load); the tables themselves are not read again
    packed = [torch.empty((hs.q6k_packed_bytes(vocab, d_model),), dtype=torch.uint8, device=dev)
              for _ in tables]
    for t, pk in zip(tables, packed):
        hs.q6k_pack(t, d_model, pk)
    hs.sync()

    def step(i=0):
        hs.project_sample_q6k_packed(hidden, norm_w, 1e-6, packed[i % 3], vocab, logits, prm, d_u,
                                     out, normed=normed)

    for i in range(args.warmup):
        step(i)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    hs.sync()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps
    ids_gpu = out.cpu().numpy()
    hs.rmsnorm(hidden, norm_w, 1e-6, normed)
    # The step above ran the arithmetic of the reference's x86 backend: for one row its integer
    # decode kernel q6k_gemv_m1 (src/backends/cpu_x86/kernel_q6k_gemv.c), for a batch
    # cpu_x86_linear_q6k_mN (linear_q6k.c:234-300: one int8 scale per row, integer dot products
    # per group of sixteen, joined as the W8A8 lane kernels of a VNNI host join them). The
    # portable arithmetic (double accumulation) is timed beside.
    x86 = m_rows == 1

    def timed(fn, tabs):
        for i in range(3):
            fn(tabs[i], i)
        with Timer() as tm:   # HIP events on the sampler's stream around the launches
            for i in range(args.steps):
                fn(tabs[i % 3], i)
        return tm.ms * 1e3 / args.steps

    portable_us = timed(lambda t, i: hs.q6k_packed_linear(t, vocab, d_model, normed, logits), packed)
    unpacked_us = timed(lambda t, i: hs.q6k_linear(t, d_model, normed, logits), tables)
    if x86:
        # geist_hip_q6k_packed_gemv_x86_rows is two launches, the activation quantiser and the
        # pass over the table; in the step the quantiser rides on the norm's launch
        kernel_us = timed(lambda t, i: hs.q6k_packed_gemv_x86(t, vocab, d_model, normed, logits),
                          packed)
        act = torch.empty((hs.q8k_act_bytes(d_model),), dtype=torch.uint8, device=dev)
        hs.q8k_quantize(normed, act)
        table_pass_us = timed(lambda t, i: hs.q6k_packed_gemv_q8k(t, vocab, d_model, act,
                                                                  logits[0]), packed)
    else:
        kernel_us = timed(lambda t, i: hs.q6k_packed_linear_x86(t, vocab, d_model, normed, logits),
                          packed)
    w_bytes = vocab * nb * 210
    achieved = w_bytes / (kernel_us * 1e-6) / 1e9
    result = {
        "metric": "sampled rows/s", "value": round(m_rows * args.steps / elapsed, 1),
        "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "Q6_K weights x int8 activations, int32 dot products, f32 accumulation",
        "data": "synthetic",
        "config": {"workload": f"lm_head_q6k_v{vocab}_d{d_model}_m{m_rows}", "rows": m_rows,
                   "n_vocab": vocab, "d_model": d_model, "temperature": 0.7, "top_k": 40,
                   "top_p": 0.9, "logit_softcap": 30.0,
                   "projection": "x86 decode kernel (q6k_gemv_m1)" if x86
                                 else "x86 batch path (cpu_x86_linear_q6k_mN)"},
        "us_per_step": round(ms * 1e3, 3), "weight_copies_rotated": 3,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": ("k_q6k_packed_gemv_x86 (+ k_q8k_quantize)" if x86 else
                                f"k_q6k_packed_gemm_x86<{min(m_rows, 8)}> (+ k_q8s_row_quantize)"),
                     "kernel_us": round(kernel_us, 3),
                     "table_passes": (m_rows + 7) // 8,
                     **({"kernel_us_table_pass_alone": round(table_pass_us, 3),
                         "frac_table_pass_alone":
                             round(w_bytes / (table_pass_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
                        if x86 else {}),
                     "kernel_us_portable_arithmetic": round(portable_us, 3),
                     "kernel_us_portable_table_as_in_file": round(unpacked_us, 3),
                     "kernel_algorithmic_bytes": w_bytes,
                     "step_algorithmic_bytes": w_bytes + m_rows * (d_model * 8 + vocab * 8 + 8)},
    }
    if not args.no_cpu:
        # CPU side on a bounded sample of the table rows, by the reference's own kernels where
        # they were compiled from its tree, else the oracle's scalar restatement; parity against
        # the strict oracle, which is the one pinned to the reference bit for bit. One row:
        # q6k_gemv_m1 (AVX2, release flags, OpenMP over the table rows). A batch:
        # w4a8_quantize_acts_row + the W8A8 kernel this host selects, over the int8 copy the
        # reference makes at load (strict flags; made before the clock starts).
        from oracle_lib import (load_oracle, load_ref_q6kgemv, load_ref_q6kmn, oracle_q6k_gemv_x86,
                                oracle_q6k_linear_x86, ref_q6k_gemv_m1, ref_q6k_mN_prepare)
        n_s = 65536 if x86 else 16384
        w_s = tables[0][:n_s].cpu().numpy()
        x_s = normed.cpu().numpy()
        kind = "port"
        if x86:
            want = oracle_q6k_gemv_x86(load_oracle(fast=False), w_s, x_s[0], d_model)[None, :]
            ref = load_ref_q6kgemv(fast=True)
            if ref is not None:
                kind = "reference"
                ref_q6k_gemv_m1(ref, w_s[:1024], x_s[0], d_model)       # threads started
                reps = 20
                t0 = time.perf_counter()
                for _ in range(reps):
                    ref_q6k_gemv_m1(ref, w_s, x_s[0], d_model)
                dt = (time.perf_counter() - t0) / reps
            else:
                lib = load_oracle(fast=True)
                t0 = time.perf_counter()
                oracle_q6k_gemv_x86(lib, w_s, x_s[0], d_model)
                dt = time.perf_counter() - t0
            hs.q6k_packed_gemv_x86(packed[0], vocab, d_model, normed, logits)
        else:
            want = oracle_q6k_linear_x86(load_oracle(fast=False), w_s, x_s, d_model)
            ref = load_ref_q6kmn()
            if ref is not None and ref.w8a8_isa_is_vnni():
                kind = "reference"
                run = ref_q6k_mN_prepare(ref, w_s, d_model)
                run(x_s)                                                # threads started
                reps = 10
                t0 = time.perf_counter()
                for _ in range(reps):
                    run(x_s)
                dt = (time.perf_counter() - t0) / reps
            else:
                lib = load_oracle(fast=True)
                t0 = time.perf_counter()
                oracle_q6k_linear_x86(lib, w_s, x_s, d_model)
                dt = time.perf_counter() - t0
            hs.q6k_packed_linear_x86(packed[0], vocab, d_model, normed, logits)
        hs.sync()
        got = logits[:, :n_s].cpu().numpy()
        result["cpu_baseline"] = {
            "value": round(m_rows / (dt * vocab / n_s), 2), "unit": "rows/s",
            "cores": int(os.environ.get("OMP_NUM_THREADS", "0") or os.cpu_count() or 1),
            "kind": kind,
            "sample": f"the projection of {m_rows} row(s) over the first {n_s} of {vocab} table rows "
                      + (("(q6k_gemv_m1: int8 activations, integer dot products"
                          + (", AVX2, mean of 20 passes)" if kind == "reference" else ", scalar C)"))
                         if x86 else
                         ("(cpu_x86_linear_q6k_mN: int8 activations, integer dot products"
                          + (", the reference's W8A8 lane kernel, mean of 10 passes)"
                             if kind == "reference" else ", scalar C)")))
                      + ", scaled to the whole table; the sampler's share of the step is not "
                        "included"}
        result["parity"] = {"logits_compared": int(want.size),
                            "logits_differ": int((got.view(np.uint32) != want.view(np.uint32)).sum())}
    result["token_ids"] = [int(t) for t in ids_gpu[:8]]
    print(json.dumps(result))
    return 0


def bench_lm_head_q4k(args, m_rows):
    """Workload lm_head_q4k[_mN]: as lm_head_q6k over a Q4_K table of the same geometry
    ([262144 x 1536], super-blocks of 144 bytes: 226 MB, read once per step and eight rows) in
    the arithmetic of the reference's x86 backend (src/backends/cpu_x86/linear_q4k.c:142-250),
    from the packed copy the head keeps (148 bytes per block); the portable kernel
    (src/backends/cpu_scalar/weight_resolve.c:82-83, 186-241 after src/formats/gguf/q4_K.c) is
    timed beside it."""
    import torch
    from geistlib_amd import HipSampler, SampleParams
    from geistlib_amd.bench_hooks import Timer
    from geistlib_amd.workloads import xorshift_units
    vocab, d_model = 262144, 1536
    nb = d_model // 256
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(13)
    hs = HipSampler(max_rows=max(m_rows, 1), max_vocab=vocab)
    tables, packed = [], []
    for _ in range(3):          # three copies (0.7 GB packed): every step's table comes from HBM
        t = torch.randint(0, 256, (vocab, nb, 144), dtype=torch.uint8, device=dev, generator=g)
        # d = binary16 0x0C6D = 2.7e-4 and dmin = 8 d in every block: logits of a few units
        t[:, :, 0], t[:, :, 1] = 0x6D, 0x0C
        t[:, :, 2], t[:, :, 3] = 0x6D, 0x18
        t = t.reshape(vocab, nb * 144).contiguous()
        pk = torch.empty((hs.q4k_packed_bytes(vocab, d_model),), dtype=torch.uint8, device=dev)
        hs.q4k_pack(t, d_model, pk)
        tables.append(t)
        packed.append(pk)
    hs.sync()
    hidden = torch.randn((m_rows, d_model), device=dev, generator=g) * 3
    norm_w = 1.0 + 0.1 * torch.randn((d_model,), device=dev, generator=g)
    u, _ = xorshift_units(7, m_rows)
    d_u = torch.from_numpy(u).to(dev)
    normed = torch.empty_like(hidden)
    logits = torch.empty((m_rows, vocab), dtype=torch.float32, device=dev)
    out = torch.empty(m_rows, dtype=torch.int32, device=dev)
    prm = SampleParams.make(temperature=0.7, top_k=40, top_p=0.9, softcap=30.0)

    def step(i=0):
        hs.project_sample_q4k_packed(hidden, norm_w, 1e-6, packed[i % 3], vocab, logits, prm, d_u,
                                     out, normed=normed)

    for i in range(args.warmup):
        step(i)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    hs.sync()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps
    ids_gpu = out.cpu().numpy()
    hs.rmsnorm(hidden, norm_w, 1e-6, normed)
    # The step above ran the arithmetic of the reference's x86 backend: for one row its integer
    # decode kernel q4kx8_gemv_m1 (src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c), for a batch
    # cpu_x86_linear_q4k_mN (linear_q4k.c:198-250: the same dot products after the batch
    # quantiser). The portable arithmetic (double accumulation) is timed beside.
    x86 = True

    def timed(fn):
        for i in range(3):
            fn(packed[i])
        with Timer() as tm:   # HIP events on the sampler's stream around the launches
            for i in range(args.steps):
                fn(packed[i % 3])
        return tm.ms * 1e3 / args.steps

    portable_us = timed(lambda t: hs.q4k_packed_linear(t, vocab, d_model, normed, logits))
    kernel_us = timed(lambda t: hs.q4k_packed_linear_x86(t, vocab, d_model, normed, logits))
    if m_rows == 1:
        # geist_hip_q4k_packed_gemv_x86_rows is two launches, the activation quantiser and the
        # pass over the table; in the step the quantiser rides on the norm's launch
        act = torch.empty((hs.q8k_row_act_bytes(d_model),), dtype=torch.uint8, device=dev)
        hs.q8k_row_quantize(normed[0], act)
        table_pass_us = timed(lambda t: hs.q4k_packed_gemv_q8k(t, vocab, d_model, act, logits[0]))
    w_bytes = vocab * nb * 144
    read_bytes = vocab * nb * 148
    achieved = w_bytes / (kernel_us * 1e-6) / 1e9
    result = {
        "metric": "sampled rows/s", "value": round(m_rows * args.steps / elapsed, 1),
        "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "Q4_K weights x int8 activations, int32 dot products, f32 accumulation",
        "data": "synthetic",
        "config": {"workload": f"lm_head_q4k_v{vocab}_d{d_model}_m{m_rows}", "rows": m_rows,
                   "n_vocab": vocab, "d_model": d_model, "temperature": 0.7, "top_k": 40,
                   "top_p": 0.9, "logit_softcap": 30.0,
                   "projection": "x86 decode kernel (q4kx8_gemv_m1)" if m_rows == 1
                                 else "x86 batch path (cpu_x86_linear_q4k_mN)"},
        "us_per_step": round(ms * 1e3, 3), "weight_copies_rotated": 3,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": f"k_q4k_packed_gemv_x86<{min(m_rows, 8)}> (+ k_q8k_row_quantize)",
                     "kernel_us": round(kernel_us, 3),
                     "table_passes": (m_rows + 7) // 8,
                     **({"kernel_us_table_pass_alone": round(table_pass_us, 3),
                         "frac_table_pass_alone":
                             round(w_bytes / (table_pass_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
                        if m_rows == 1 else {}),
                     "kernel_us_portable_arithmetic": round(portable_us, 3),
                     "kernel_algorithmic_bytes": w_bytes,
                     "packed_bytes_read": read_bytes,
                     "step_algorithmic_bytes": w_bytes + m_rows * (d_model * 8 + vocab * 8 + 8)},
    }
    if not args.no_cpu:
        # CPU side on a bounded sample of the table rows: the reference's own kernels over the
        # table its own repacker interleaves (release flags, OpenMP over the row tiles) where
        # they were compiled from the reference's tree -- q4kx8_gemv_m1 for one row,
        # quantize_q8_Kx4 + q4kx8_gemm_avx512 for a batch of a multiple of 4 rows, the decode
        # kernel row by row for the others, as cpu_x86_linear_q4k_mN calls them --, else the
        # oracle's scalar restatement; parity against the strict oracle, which is the one pinned
        # to the reference bit for bit.
        from oracle_lib import (load_oracle, load_ref_q4kgemv, oracle_q4k_linear_x86,
                                Q4KX8_BLOCK_BYTES, Q8KX4_BLOCK_BYTES)
        import ctypes as C
        n_s = 65536
        w_s = tables[0][:n_s].cpu().numpy()
        x_s = np.ascontiguousarray(normed.cpu().numpy())
        kind = "port"
        want = oracle_q4k_linear_x86(load_oracle(fast=False), w_s, x_s, d_model)
        ref = load_ref_q4kgemv(fast=True)
        if ref is not None:
            kind = "reference"
            blob = np.zeros(n_s // 8 * nb * Q4KX8_BLOCK_BYTES + 64, dtype=np.uint8)
            ref.q4k_to_q4kx8_matrix(d_model, n_s, w_s.ctypes.data_as(C.c_void_p),
                                    blob.ctypes.data_as(C.c_void_p))      # once, as at load
            yr = np.empty((m_rows, n_s), dtype=np.float32)
            fp = C.POINTER(C.c_float)
            acts = np.zeros(max(m_rows // 4, 1) * nb * Q8KX4_BLOCK_BYTES + 64, dtype=np.uint8)

            def cpu_call():
                if m_rows % 4 != 0:
                    for i in range(m_rows):
                        ref.q4kx8_gemv_m1(n_s, d_model, x_s[i].ctypes.data_as(fp),
                                          blob.ctypes.data_as(C.c_void_p), yr[i].ctypes.data_as(fp))
                    return
                for mt in range(m_rows // 4):
                    ref.quantize_q8_Kx4(d_model, x_s[4 * mt:4 * mt + 4].ctypes.data_as(fp),
                                        C.c_void_p(acts.ctypes.data + mt * nb * Q8KX4_BLOCK_BYTES))
                ref.q4kx8_gemm_avx512(m_rows, n_s, d_model, acts.ctypes.data_as(C.c_void_p),
                                      blob.ctypes.data_as(C.c_void_p), yr.ctypes.data_as(fp))

            cpu_call()                                                      # threads started
            reps = 20
            t0 = time.perf_counter()
            for _ in range(reps):
                cpu_call()
            dt = (time.perf_counter() - t0) / reps
        else:
            lib = load_oracle(fast=True)
            t0 = time.perf_counter()
            oracle_q4k_linear_x86(lib, w_s, x_s, d_model)
            dt = time.perf_counter() - t0
        hs.q4k_packed_linear_x86(packed[0], vocab, d_model, normed, logits)
        hs.sync()
        got = logits[:, :n_s].cpu().numpy()
        result["cpu_baseline"] = {
            "value": round(m_rows / (dt * vocab / n_s), 2), "unit": "rows/s",
            "cores": int(os.environ.get("OMP_NUM_THREADS", "0") or os.cpu_count() or 1),
            "kind": kind,
            "sample": f"the projection of {m_rows} row(s) over the first {n_s} of {vocab} table rows "
                      + ("(" + ("q4kx8_gemv_m1" if m_rows % 4 else "quantize_q8_Kx4 + q4kx8_gemm_avx512")
                         + ": int8 activations, integer dot products"
                         + (", the reference's vector kernels, mean of 20 passes)"
                            if kind == "reference" else ", scalar C)"))
                      + ", scaled to the whole table; the sampler's share of the step is not "
                        "included"}
        result["parity"] = {"logits_compared": int(want.size),
                            "logits_differ": int((got.view(np.uint32) != want.view(np.uint32)).sum())}
    result["token_ids"] = [int(t) for t in ids_gpu[:8]]
    print(json.dumps(result))
    return 0


def bench_lm_head_spec(args):
    """Workload lm_head_spec: the tail of a greedy decode step for BitNet-2B-4T's geometry through
    the reference's speculative output head (forward/spec_head.c): RMS norm of the hidden row,
    rough scores of the 128256 rows over a 640-dimension int8 sketch (82 MB), the 1024 best-ranked
    rows scored exactly against the F16 table, the best of them. A step is one such tail; the
    dominant kernel is the int8 projection over the sketch."""
    import torch
    from geistlib_amd import HipSampler, SpecResult
    vocab, d_model = 128256, 2560
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    hs = HipSampler(max_rows=1, max_vocab=vocab)
    # three tables and their sketches (3 x 739 MB): every step's sketch and finalist rows come
    # from HBM
    tables = [(torch.randn((vocab, d_model), device=dev, generator=g) * 0.05).to(torch.float16)
              for _ in range(3)]
    heads = [hs.spec_head_build(t) for t in tables]
    views = [hs.spec_head_view(sh) for sh in heads]
    sd, topk = views[0].sketch_dim, views[0].topk
    hidden = torch.randn((1, d_model), device=dev, generator=g) * 3
    norm_w = 1.0 + 0.1 * torch.randn((d_model,), device=dev, generator=g)
    normed = torch.empty_like(hidden)
    res = torch.zeros(6, dtype=torch.int32, device=dev)

    def step(i=0):
        hs.spec_head_try_hidden(heads[i % len(heads)], hidden, norm_w, 1e-6, normed, res)

    for i in range(args.warmup):
        step(i)
    hs.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    hs.sync()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps
    got = SpecResult.from_buffer_copy(res.cpu().numpy().tobytes())
    # the projection over the sketch alone
    act = torch.randint(-127, 128, (1, sd), device=dev, generator=g).to(torch.float32)
    rough = torch.empty((1, vocab), dtype=torch.float32, device=dev)
    from geistlib_amd.bench_hooks import Timer
    sketches = [_DevPtr(v.d_sketch, (vocab, sd)) for v in views]
    row_scales = [_DevPtr(v.d_row_scale, (vocab,)) for v in views]
    for i in range(len(views)):
        hs.q8w_gemv(sketches[i], row_scales[i], act, rough)
    with Timer() as tm:
        for i in range(args.steps):
            hs.q8w_gemv(sketches[i % len(views)], row_scales[i % len(views)], act, rough)
    kernel_us = tm.ms * 1e3 / args.steps
    k_bytes = vocab * sd + vocab * 4
    achieved = k_bytes / (kernel_us * 1e-6) / 1e9
    result = {
        "metric": "sampled rows/s", "value": round(args.steps / elapsed, 1), "unit": "rows/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 sketch x int8 activations (exact in f32), f16 x f32 finalists",
        "data": "synthetic",
        "config": {"workload": f"lm_head_spec_v{vocab}_d{d_model}", "rows": 1, "n_vocab": vocab,
                   "d_model": d_model, "sketch_dim": sd, "finalists": topk, "temperature": 0.0},
        "us_per_step": round(ms * 1e3, 3), "weight_copies_rotated": len(tables),
        "finalists_scored": got.n_listed,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "k_q8w_gemv", "kernel_us": round(kernel_us, 3),
                     "kernel_algorithmic_bytes": k_bytes,
                     "step_algorithmic_bytes": k_bytes + vocab * 8 + got.n_listed * d_model * 2
                     + d_model * 8},
    }
    if not args.no_cpu:
        # the oracle's restatement of spec_head.c on this host's cores (its rough-score loop runs
        # on OpenMP threads as the reference's does; heap and finalists are serial there too)
        from oracle_lib import Oracle
        o = Oracle()
        j = (args.steps - 1) % len(tables)
        wt = tables[j].cpu().numpy().view(np.uint16)
        sh = o.spec_head_build(wt)
        x_host = normed.cpu().numpy()[0]
        reps, t_used = 0, 0.0
        while reps < 20 and t_used < 10.0:
            t1 = time.perf_counter()
            want = sh.try_row(x_host)
            t_used += time.perf_counter() - t1
            reps += 1
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or 10 ** 6)
        result["cpu_baseline"] = {"value": round(reps / t_used, 2), "unit": "rows/s", "cores": cores,
                                  "kind": "port",
                                  "sample": f"{reps} calls of the sketch head on one normed row "
                                            "(sketch built beforehand, no norm)"}
        dense = o.f16_gemv(wt, x_host)
        result["parity"] = {"rows": 1, "ids_differ": int(got.token != want["token"]),
                            "cutoff_identical": bool(got.cutoff == want["cutoff"]),
                            "token_is_dense_argmax": bool(got.token == int(np.argmax(dense))),
                            "winner_logit_bit_identical": bool(
                                np.float32(got.best_exact).view(np.uint32)
                                == dense[got.token].view(np.uint32))}
    for sh_ in heads:
        hs.spec_head_destroy(sh_)
    print(json.dumps(result))


def bench_whole_row_walk(args):
    """Workload whole_row_walk: top-p rows whose kept prefix is tens of thousands of entries (flat
    rows at temperature 1: logits N(0, 0.5^2), top-p 0.9), which neither the thread-maxima
    shortcut nor the candidate list can serve: every row is walked in full
    (src/engine/sampler.c:246-304 sorts and walks it). Timed per step for 1, 16 and 64 rows of
    128256 with the walk by one workgroup per row and spread over the workgroups of the row's
    chunks (geist_hip_sampler_set_whole_row_walk), the steps reading four copies of the batch in
    turn; the ids of the two forms are compared with each other and, without --no-cpu, the
    16-row batch with the oracle."""
    import torch
    from geistlib_amd import HipSampler, SampleParams
    from geistlib_amd.bench_hooks import Timer
    dev = torch.device("cuda:0")
    n = 128256
    prm = SampleParams.make(temperature=1.0, top_p=0.9)
    legs, ids16, x16, u16 = {}, None, None, None
    for rows in (1, 16, 64):
        hs = HipSampler(max_rows=rows, max_vocab=n)
        g = torch.Generator(device=dev)
        g.manual_seed(100 + rows)
        xs = [torch.randn((rows, n), device=dev, generator=g) * 0.5 for _ in range(4)]
        u = torch.rand(rows, device=dev, generator=g)
        out = torch.empty(rows, dtype=torch.int32, device=dev)
        got = {}
        for name, mode in (("one_workgroup", 2), ("spread", 1)):
            hs.set_whole_row_walk(mode)
            for i in range(8):
                hs.sample(HipSampler.rows(xs[i % 4]), prm, u, out)
            hs.sync()
            steps = max(8, min(args.steps, 100))
            with Timer() as tm:
                for i in range(steps):
                    hs.sample(HipSampler.rows(xs[i % 4]), prm, u, out)
            hs.sample(HipSampler.rows(xs[0]), prm, u, out)
            hs.sync()
            got[name] = out.cpu().numpy().tolist()
            legs[f"rows{rows}_{name}_us_per_step"] = round(tm.ms * 1e3 / steps, 2)
            legs[f"rows{rows}_{name}_paths"] = sorted(set(hs.row_paths(rows).tolist()))
        legs[f"rows{rows}_ids_equal"] = got["one_workgroup"] == got["spread"]
        if rows == 16:
            ids16, x16, u16 = got["spread"], xs[0].cpu().numpy(), u.cpu().numpy()
        hs.close()
    result = {
        "metric": "sampled rows/s", "value": round(16 / (legs["rows16_spread_us_per_step"] * 1e-6), 1),
        "unit": "rows/s", "n_gpus": 1, "steps": max(8, min(args.steps, 100)), "warmup": 8,
        "ms_per_step": round(legs["rows16_spread_us_per_step"] * 1e-3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "whole_row_walk_b16_v128256", "rows": 16, "n_vocab": n,
                   "temperature": 1.0, "top_p": 0.9, "logits": "N(0, 0.5^2)"},
        "legs": legs,
    }
    if not args.no_cpu:
        from oracle_lib import Oracle
        o = Oracle(fast=True)
        want = [int(o.top_p_u(x16[r], 0.9, 1.0, float(u16[r]))[0]) for r in range(16)]
        result["parity"] = {"rows": 16, "ids_differ": int(sum(a != b for a, b in zip(ids16, want)))}
    print(json.dumps(result))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="cfg2_pen")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cold-only", action="store_true",
                    help="skip the cache-resident legs and the latency probe, so that every launch "
                         "of the run streams its logits from HBM (for rocprofv3 runs whose "
                         "per-kernel averages are to be compared with roofline.kernel_us)")
    ap.add_argument("--fast-sums", action="store_true",
                    help="geist_hip_sampler_set_sums(GEIST_HIP_SUMS_FAST): the sums of exponentials "
                         "from the hardware's 2^z (the tolerance of the sampling contract used; "
                         "off by default, and never the headline figure)")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the legs that time configurations 1, 3, 4 and 5 beside the headline "
                         "workload")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="instead of sampling, run a plain device copy of the logit buffer "
                         "(a kernel of known traffic, for scaling rocprof's FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: rows are independent and this build has no "
                         "multi-GPU path (run with --gpus 1)")

    import torch
    from geistlib_amd import HipSampler, SampleParams
    if not torch.cuda.is_available():
        raise SystemExit("no GPU visible: the sampling path has no CPU fallback")

    if args.workload == "whole_row_walk":
        return bench_whole_row_walk(args)
    if args.workload == "lm_head_spec":
        return bench_lm_head_spec(args)
    if args.workload.startswith("lm_head_q6k"):
        m = int(args.workload.split("_m")[1]) if "_m" in args.workload else 1
        return bench_lm_head_q6k(args, m)
    if args.workload.startswith("lm_head_q4k"):
        m = int(args.workload.split("_m")[1]) if "_m" in args.workload else 1
        return bench_lm_head_q4k(args, m)
    if args.workload.startswith("lm_head"):
        m = int(args.workload.split("_m")[1]) if "_m" in args.workload else 1
        return bench_lm_head(args, m, q8=args.workload.startswith("lm_head_q8"))
    w = build_workload(args.workload)
    if args.workload == "cfg5":
        return bench_spec(w, args)
    dev = torch.device("cuda:0")
    d_logits = torch.from_numpy(w.logits).to(dev)
    d_u = torch.from_numpy(w.uniforms).to(dev)
    d_h = torch.from_numpy(w.history).to(dev) if w.history is not None else None
    d_hl = torch.from_numpy(w.history_len).to(dev) if w.history is not None else None
    d_out = torch.empty(w.rows, dtype=torch.int32, device=dev)
    hs = HipSampler(max_rows=w.rows, max_vocab=w.n_vocab)
    if args.fast_sums:
        hs.set_sums(fast=True)
    rows = HipSampler.rows(d_logits, d_h, d_hl)
    prm = SampleParams.make(temperature=w.temperature, top_k=w.top_k, top_p=w.top_p,
                            min_p=w.min_p, rep=w.rep, freq=w.freq, pres=w.pres)

    if args.calibrate_copy:
        dst = torch.empty_like(d_logits)
        for _ in range(args.steps):
            dst.copy_(d_logits)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": d_logits.numel() * 4,
                          "calibrate_copy_bytes_written": d_logits.numel() * 4,
                          "launches": args.steps}))
        return

    # Inputs resident in HBM, not in the caches: the steps rotate over copies of the batch that
    # together exceed the 256 MB Infinity Cache (plus the L2s) more than twice, so every step
    # streams its logits from HBM. One buffer used over and over would stay cache-resident and
    # the streaming kernel would run above the HBM rate.
    n_copies = min(64, max(2, -(-COLD_WORKING_SET // (d_logits.numel() * 4))))
    copies = [d_logits] + [d_logits.clone() for _ in range(n_copies - 1)]
    rows_cold = [HipSampler.rows(c, d_h, d_hl) for c in copies]

    def step(i=0):
        hs.sample(rows_cold[i % n_copies], prm, d_u, d_out)

    from geistlib_amd import bench_hooks as bh

    # The cold legs tell the sampler what they are: logits that come from HBM and are read once
    # (GEIST_HIP_LOGITS_STREAMED). The cache-resident legs run with the default hint.
    hs.set_logits_hint(True)
    # Untimed and reported: one pass over every copy before the counted warm-up, so that a short
    # run (the driver's 20 steps) does not time first touches of 690 MB and idle clocks.
    prewarm = 3 * n_copies
    for i in range(prewarm):
        step(i)
    hs.sync()
    for i in range(args.warmup):
        step(i)
    hs.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    hs.sync()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    ids_gpu = d_out.cpu().numpy()

    # the same with one buffer: logits that the caches still hold from the step before (in a
    # decoder the lm_head has just written them)
    ms_resident = None
    if not args.cold_only:
        hs.set_logits_hint(False)
        for _ in range(args.warmup):
            step(0)
        hs.sync()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            step(0)
        hs.sync()
        ms_resident = (time.perf_counter() - t1) * 1e3 / args.steps

    # the logit-streaming kernel on its own: HIP events on the sampler's stream around K
    # back-to-back launches of that kernel (same configuration), again over the rotating copies
    hs.set_logits_hint(True)
    kernel_us, kernel_name = bh.time_stream_kernel(hs, rows_cold, prm, d_u, d_out, args.steps)
    # where the step is one launch (scan and row-final together), the scan kernel of the
    # two-launch form on its own as well: the rate at which the logits are streamed
    scan_alone_us = scan_alone_name = None
    if kernel_name == "k_cand_scan_final":
        hs.one_launch_topk(False)
        scan_alone_us, scan_alone_name = bh.time_stream_kernel(hs, rows_cold, prm, d_u, d_out,
                                                               args.steps)
        hs.one_launch_topk(True)
    # calibration: a kernel that only reads the same rows with the same geometry
    plain_us = bh.time_plain_read(rows_cold, args.steps, streamed=True)
    hs.set_logits_hint(False)
    plain_us_resident = None if args.cold_only else bh.time_plain_read([rows], args.steps,
                                                                       streamed=False)
    kernel_us_resident = (None if args.cold_only
                          else bh.time_stream_kernel(hs, [rows], prm, d_u, d_out, args.steps)[0])
    hs.set_logits_hint(True)

    # one-step latency: enqueue + wait, median
    lat = []
    for i in range(0 if args.cold_only else 200):
        t1 = time.perf_counter()
        step(i)
        hs.sync()
        lat.append((time.perf_counter() - t1) * 1e6)
    lat.sort()
    # the same with the ids landing in page-locked host memory (the kernels write them there in
    # place): from the call to token ids the host can read, no copy in between
    lat_host = []
    if not args.cold_only:
        out_host = hs.host_buffer(w.rows * 4)
        ids_host = out_host.view(np.int32)
        for i in range(200):
            t1 = time.perf_counter()
            hs.sample(rows_cold[i % n_copies], prm, d_u, out_host)
            hs.sync()
            lat_host.append((time.perf_counter() - t1) * 1e6)
        lat_host.sort()
        assert ids_host.tolist() == d_out.cpu().numpy().tolist()
        # the same measured from C, call to ids readable on the host (clock_gettime around
        # geist_hip_sample_rows + the wait), first with the wait for the stream, then with the
        # sampler telling the host when the ids are written (geist_hip_sampler_notify_ids /
        # _wait_ids): the figure a caller of the synchronous entry points sees
        lat_c_sync = sorted(bh.step_latency(hs, rows_cold, prm, d_u, out_host, 200, wait_ids=False))
        hs.notify_ids(True)
        bh.step_latency(hs, rows_cold, prm, d_u, out_host, 20, wait_ids=True)
        lat_c_wait = sorted(bh.step_latency(hs, rows_cold, prm, d_u, out_host, 200, wait_ids=True))
        # ... and on one buffer over and over, which stays cache-resident as logits are right
        # after the projection that wrote them (with the default kind of load)
        hs.set_logits_hint(False)
        bh.step_latency(hs, [rows], prm, d_u, out_host, 20, wait_ids=True)
        lat_c_wait_res = sorted(bh.step_latency(hs, [rows], prm, d_u, out_host, 200, wait_ids=True))
        hs.set_logits_hint(True)
        hs.notify_ids(False)
        assert ids_host.tolist() == d_out.cpu().numpy().tolist()
        out_host.close()

    alg_bytes = w.algorithmic_bytes()
    # the streaming kernel's own share of those bytes: every logit once
    kernel_bytes = w.rows * w.n_vocab * 4
    scan_bytes = kernel_bytes
    if kernel_name in ("k_cand_scan_final", "k_temperature_draw"):
        kernel_bytes = alg_bytes  # the kernel is the whole step
    achieved = kernel_bytes / (kernel_us * 1e-6) / 1e9
    # (the counter runs were taken with the one-launch kernel)
    traffic = (PROFILED_TRAFFIC.get(w.name, (None, None)) if kernel_name == "k_cand_scan_final"
               else (None, None))
    result = {
        "metric": "sampled rows/s",
        "value": round(w.rows * args.steps / elapsed, 1),
        "unit": "rows/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": w.name, "sums": "fast" if args.fast_sums else "exact",
                   "rows": w.rows, "n_vocab": w.n_vocab,
                   "temperature": w.temperature, "top_k": w.top_k, "top_p": w.top_p,
                   "min_p": w.min_p, "penalties": [w.rep, w.freq, w.pres],
                   "history_per_row": 0 if w.history is None else int(w.history.shape[1])},
        "us_per_step": round(ms_per_step * 1e3, 3),
        "us_per_step_cache_resident": None if ms_resident is None else round(ms_resident * 1e3, 3),
        "rows_per_s_cache_resident": None if ms_resident is None else round(
            w.rows / (ms_resident * 1e-3), 1),
        "input_copies_rotated": n_copies,
        "prewarm_steps": prewarm,
        "step_latency_us_median": round(lat[len(lat) // 2], 2) if lat else None,
        "step_latency_from_c_stream_wait_us_median": (round(lat_c_sync[len(lat_c_sync) // 2], 2)
                                                      if lat_host else None),
        "step_latency_from_c_ids_on_host_us_median": (round(lat_c_wait[len(lat_c_wait) // 2], 2)
                                                      if lat_host else None),
        "step_latency_from_c_ids_on_host_us_p90": (round(lat_c_wait[len(lat_c_wait) * 9 // 10], 2)
                                                   if lat_host else None),
        "step_latency_from_c_ids_on_host_cache_resident_us_median": (
            round(lat_c_wait_res[len(lat_c_wait_res) // 2], 2) if lat_host else None),
        "step_latency_ids_on_host_us_median": (round(lat_host[len(lat_host) // 2], 2)
                                               if lat_host else None),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic[0], "traffic_source": traffic[1],
                     "kernel": kernel_name,
                     "kernel_us": round(kernel_us, 3),
                     "kernel_us_cache_resident": None if kernel_us_resident is None else round(
                         kernel_us_resident, 3),
                     "plain_read_us": round(plain_us, 3),
                     "plain_read_us_cache_resident": None if plain_us_resident is None else round(
                         plain_us_resident, 3),
                     "kernel_algorithmic_bytes": kernel_bytes,
                     "step_algorithmic_bytes": alg_bytes,
                     "step_frac": round(alg_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
    }
    if w.top_k:
        result["topk_paths"] = topk_path_counts(hs, rows_cold, prm, d_u, d_out, w.rows)
    if scan_alone_us is not None:
        result["roofline"]["scan_kernel_of_two_launch_form"] = {
            "kernel": scan_alone_name, "kernel_us": round(scan_alone_us, 3),
            "frac": round(scan_bytes / (scan_alone_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
    if not args.no_cpu:
        base, ids_cpu = cpu_baseline(w)
        result["cpu_baseline"] = base
        if ids_cpu is not None:
            result["parity"] = {"rows": int(w.rows),
                                "ids_differ": int(np.sum(ids_cpu != ids_gpu))}
    if args.workload == "cfg2_pen" and not args.cold_only and not args.no_configs:
        # the headline run also carries the other four configurations' figures
        hs.close()
        del copies, rows_cold
        torch.cuda.empty_cache()
        result["configs"] = time_other_configs()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
