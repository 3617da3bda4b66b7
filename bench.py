#!/usr/bin/env python3
"""LRQK decode benchmark on one MI355X.

A "step" is one decode step of ONE layer: ring append, factor update, proxy-score scan over
all cached tokens, top-k, hit/miss diff, miss fetch from the pinned host store, and exact
attention over the k + lite active tokens.  Default workload: Llama-3-8B attention shape at a
128K-token context (32 q / 8 kv heads, d 128, bf16, r 32, k 2048, lite 64, max_iter (2,2)).

Prints ONE JSON line.  `value` is microseconds per layer-step with all inputs resident (the
per-step q,k,v are pre-staged in HBM; the host store is pinned host memory by definition
of the path).  `roofline` is the proxy-score kernel (the dominant HBM stream): algorithmic
bytes Hq * m * r * elem per launch over its HIP-event duration.  `cpu_baseline` times the CPU
oracle on a few steps continued from the same state.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# HBM bytes per launch of the proxy-score kernel read from hardware counters (rocprofv3 --pmc FETCH_SIZE, then
# WRITE_SIZE, each scaled by what the same counter reads for a 256 MiB device copy: x2.000 and x1.000), per
# workload at its default context (the scaling factors come from this library's own probe kernels of known size in
# the same runs).  The summary of those runs is kept under profiles/.
# Keyed by (workload, score index in use): with the index the kernel is score_prefilter_kernel and reads the
# 8-bit copy (34 bytes per row) plus the rows it rescores; without it score_filter_kernel reads A_K itself.
MEASURED_TRAFFIC = {
    ("llama8b_128k_bf16", True): {"bytes": (78875.8 * 2.000 + 1007.1 * 1.000) * 1024, "rows_rescored_in_that_run": 153723,
                                  "profile": "profiles/decode_step_llama8b_128k_hbm_traffic_and_sq_counters.md"},
    ("llama8b_128k_bf16", False): {"bytes": (131110.0 * 2.000 + 1060.2 * 1.000) * 1024, "rows_rescored_in_that_run": 0,
                                   "profile": "profiles/decode_step_llama8b_128k_hbm_traffic_and_sq_counters.md "
                                              "(an earlier build's run of --no-score-index)"}}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=512)  # the count the 128K configuration is quoted on
    p.add_argument("--warmup", type=int, default=16)
    p.add_argument("--workload", default="llama8b_128k_bf16")
    p.add_argument("--context", type=int, default=None, help="override the context length")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--cpu-steps", type=int, default=160,
                   help="decode mode: oracle steps timed for cpu_baseline (about 12 s of host work at the 128K "
                        "configuration); the other modes only ask whether it is 0 (= no cpu_baseline)")
    p.add_argument("--cpu-threads", type=int, default=0,
                   help="0 = every core this process may use (affinity mask, OMP_NUM_THREADS where the host is shared)")
    p.add_argument("--min-timed", type=int, default=512,
                   help="decode mode: when --steps is smaller than this, `value` is timed over this many steps in a "
                        "second region (the region of exactly --steps steps is reported beside it)")
    p.add_argument("--event-steps", type=int, default=64,
                   help="decode mode: steps of the pass after the timed regions in which every proxy-score launch of "
                        "the first copy sits between two HIP events (no timed region has an event inside a step)")
    p.add_argument("--also", default="auto", choices=["auto", "on", "off"],
                   help="decode mode: add compact results of the other configurations (32K decode, four sequences, "
                        "prefill factorisation, full decoder) under the `also` key; auto = for the default workload "
                        "with no overrides")
    p.add_argument("--no-also-decoder", dest="also_decoder", action="store_false",
                   help="leave the full decoder out of `also`")
    p.add_argument("--also-budget-s", type=float, default=150.0,
                   help="the full decoder of `also` is skipped when the run has already taken this long")
    p.add_argument("--no-probe-sweep", action="store_true",
                   help="skip the sweep over the variants of the plain read kernel")
    p.add_argument("--no-attn", action="store_true", help="leave the attention kernel out of the step")
    p.add_argument("--variant", default="default", choices=["default", "no_hit_miss"])
    p.add_argument("--fetch", default="direct", choices=["direct", "staged"],
                   help="miss fetch: the kernel reads the pinned store itself, or host gather + hipMemcpyAsync")
    p.add_argument("--no-score-index", action="store_true",
                   help="scan the bf16 A_K rows directly instead of their 8-bit score index")
    p.add_argument("--factor-state", action="store_true",
                   help="run every step's factor update in fp64 from the state kept between steps instead of over the "
                        "active rows in fp32 (adds a launch per step that brings the state up to date)")
    p.add_argument("--victim-rows", type=int, default=-1,
                   help="rows per head of the device-side cache of evicted K/V rows (-1: 4 k, 0: off)")
    p.add_argument("--mode", default="decode", choices=["decode", "prefill_als", "decoder"],
                   help="prefill_als: time the prefill factorisation alone (workload llama8b_32k_prefill_als unless "
                        "--workload is given); a step is one whole factorisation.  decoder: greedy decoding with a "
                        "full Llama-3-8B-shaped stack around the cache (end-to-end tokens/s)")
    p.add_argument("--layers", type=int, default=32, help="decoder mode: number of layers")
    p.add_argument("--batch", type=int, default=4, help="decoder mode: sequences")
    p.add_argument("--prompt", type=int, default=65536, help="decoder mode: prompt tokens per sequence")
    p.add_argument("--new-tokens", type=int, default=128, help="decoder mode: tokens decoded per sequence")
    p.add_argument("--max-iter", type=int, default=0,
                   help="decode mode: iterations of the factor update per step and at the prompt instead of the workload's "
                        "(the reference's throughput script runs 8, tps_estimate.py:20-29); with --tol")
    p.add_argument("--tol", type=float, default=1e-8, help="stopping tolerance used with --max-iter")
    p.add_argument("--rank", type=int, default=0, help="decode mode: r instead of the workload's")
    p.add_argument("--topk", type=int, default=0, help="decode mode: active tokens k instead of the workload's")
    p.add_argument("--lite", type=int, default=0, help="decode mode: recent-token window instead of the workload's")
    p.add_argument("--data-rank", type=int, default=0,
                   help="decode mode: rank of the synthetic queries / keys before noise instead of the workload's 32 "
                        "(a factorisation of rank r on data of lower rank has directions that hold only noise)")
    p.add_argument("--seqs", type=int, default=0,
                   help="decode mode: sequences stepped together (the batch of the layer-step; 0 = the workload's "
                        "own, 1 for the 128K configuration); value stays the time of one layer-step of the whole batch")
    p.add_argument("--context-scale", type=float, default=0.0,
                   help="decoder mode: length of a fixed direction added to every token embedding (in embedding "
                        "lengths); > 0 makes successive queries correlated, as a trained model's are (random weights and "
                        "random ids alone give unrelated queries and a hit rate of k / l)")
    p.add_argument("--settle", type=int, default=512,
                   help="decode mode: further untimed steps before the warm-up steps.  The first process on a box "
                        "enqueues its first few hundred steps several times slower than later ones (cold host-side "
                        "launch path), slower than the GPU executes them, and 16 warm-up steps do not get past that")
    p.add_argument("--rotate", type=int, default=4,
                   help="decode mode: step this many independent copies of the layer's state in turn (as the layers "
                        "of a decoder do), so that no copy finds its buffers in the 256 MB last-level cache; the "
                        "value is the time per layer-step; kernel timing is taken from the first copy.  1 = one "
                        "copy stepped back to back (its score index stays in that cache)")
    p.add_argument("--warm-steps", type=int, default=128,
                   help="decode mode: after the timed region, step the first copy alone this many times and report "
                        "that (cache-warm) time per step as a secondary figure; 0 = skip")
    p.add_argument("--probe-mb", type=int, default=2048,
                   help="decode mode: size of the buffer the sweep of plain read kernels runs over (the default read / "
                        "copy pair runs over at most 1024 MiB); 0 = no probes")
    p.add_argument("--calib-copy-mb", type=int, default=0,
                   help="after the timed region, run one plain device copy of this many MiB (a known-size "
                        "kernel to scale hardware counters by)")
    return p.parse_args()


def oracle_from_engine(eng, w, threads):
    """A CPU oracle layer continued from the engine's current state."""
    from oracle import lrqk_oracle as orc
    orc.set_threads(threads)
    o = orc.OracleLayer(num_lite_tokens=w.lite_tokens, attn_topk=w.num_active_tokens, num_key_value_groups=w.groups,
                        r=w.r, max_iter=w.max_iter, tol=w.tol, capacity=eng._A_K.capacity,
                        compute_dtype=torch.float32, no_hit_miss=eng.no_hit_miss)
    torch.cuda.synchronize()
    o.B_Q, o.B_K = eng.B_Q.cpu(), eng.B_K.cpu()
    o._A_K.data, o._A_K.capacity, o._A_K.current_len = eng._A_K.data.cpu(), eng._A_K.capacity, eng._A_K.current_len
    o._A_K.dtype = eng._A_K.data.dtype
    o.KVcpu.data, o.KVcpu.capacity, o.KVcpu.current_len = eng.KVcpu.data.clone(), eng.KVcpu.capacity, eng.KVcpu.current_len
    o.KVcpu.dtype = eng.KVcpu.data.dtype
    o.Kgpu, o.Vgpu = eng.Kgpu.cpu(), eng.Vgpu.cpu()
    o.hit_indices = eng.hit_indices.cpu()
    o.lite_indices, o.lite_len = list(eng.lite_indices), eng.lite_len
    o.current_len, o.prefill_length = eng.current_len, eng.prefill_length
    return o, orc


FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix peak, published
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak, published


def prefill_als(a):
    """Times lrqk_als_prefill on synthetic low-rank + noise Q, K and reports fit residuals."""
    from lrqk_amd import synth, ops
    dev = torch.device("cuda:0")
    w = synth.WORKLOADS[a.workload if a.workload != "llama8b_128k_bf16" else "llama8b_32k_prefill_als"]
    l = a.context or w.context
    Q, K, V, bases, gen = synth.prompt_qkv(w, a.seed, l, device=dev)
    del V
    A0 = synth.init_factors(w, l, a.seed + 1, device=dev)
    ws = ops.Workspace()
    iters, tol = w.max_iter[0], w.tol[0]
    steps, warm = min(a.steps, 8), min(a.warmup, 2)
    res = None
    times = []
    for i in range(warm + steps):
        aq, ak = A0[0].clone(), A0[1].clone()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        res = ops.als_prefill(ws, Q, K, aq, ak, iters, tol)
        torch.cuda.synchronize()
        if i >= warm:
            times.append(time.perf_counter() - t0)
    ms = sum(times) / len(times) * 1e3
    AQ, BQ, AK, BK = res
    g = w.num_heads // w.num_kv_heads
    # residuals head by head (the fp32 copy of all heads at once would double the footprint)
    num_k = den_k = num_q = den_q = 0.0
    for h in range(w.num_heads):
        Kh = K[:, h // g].float()
        Qh = Q[:, h].float()
        num_k += float((Kh - AK[:, h] @ BK[:, h]).pow(2).sum()); den_k += float(Kh.pow(2).sum())
        num_q += float((Qh - AQ[:, h] @ BQ[:, h]).pow(2).sum()); den_q += float(Qh.pow(2).sum())
    bh = w.batch * w.num_heads
    r, d = w.r, w.head_dim
    cpu = None
    if a.cpu_steps > 0:
        # the oracle's fp32 run of the same factorisation on a few heads, scaled to all heads
        from oracle import lrqk_oracle as orc
        threads, host = host_threads(a)
        torch.set_num_threads(threads)
        hs = list(range(0, w.num_heads, max(1, w.num_heads // 4)))[:4]
        Qc = Q[:, hs].float().cpu()
        Kc = K[:, [h // g for h in hs]].float().cpu()
        a0, k0 = A0[0][:, hs].cpu(), A0[1][:, hs].cpu()
        orc.als_prefill_w1(Qc[:, :1], Kc[:, :1], a0[:, :1], k0[:, :1], 1, tol)   # untimed warm-up
        t0 = time.perf_counter()
        orc.als_prefill_w1(Qc, Kc, a0, k0, iters, tol)
        cpu_ms = (time.perf_counter() - t0) * 1e3 * (w.batch * w.num_heads / len(hs))
        cpu = {"value": round(cpu_ms, 1), "unit": "ms", "cores": threads, "kind": "port",
               "sample": f"fp32 torch-CPU factorisation of {len(hs)} of the {w.num_heads} heads at the full length "
                         f"on {threads} threads, scaled to all heads"}
        cpu.update(host)
    # one pass = apply (2 l d r) + Grams (2 l r (r + d)); 2 initial Gram passes + 2 passes per iteration
    flops = bh * (2 * 2.0 * l * r * (r + d) + iters * 2 * (2.0 * l * d * r + 2.0 * l * r * (r + d)))
    e = 2 if w.dtype == torch.bfloat16 else 4
    # HBM bytes: every pass reads X once; apply passes read and write A (fp32), Gram passes read A
    bytes_ = bh * ((2 + 2 * iters) * l * d * e + 2 * l * r * 4 + iters * 2 * 2 * l * r * 4)
    tf = flops / (ms * 1e-3) / 1e12
    bkv = w.batch * w.num_kv_heads
    if e == 2 and d == 128 and r <= 32 and not os.environ.get("LRQK_PREFILL_ROWWISE"):
        # bf16 rows of 128 elements: the iterations run on d x d Gram matrices (fp64, 32 small independent problems),
        # and the long axis is read a fixed number of times whatever the iteration count: Q twice (sums over the
        # given factors together with Q^T Q; the final A_Q = Q Mq), K three times, once per kv head (sums over the
        # given factors, K^T K, the final A_K = K Mk).  HBM bytes: those + the initial factors read + the final
        # factors written (fp32).
        bytes_g = (2.0 * bh + 3.0 * bkv) * l * d * e + 4.0 * bh * l * r * 4
        gbs = bytes_g / (ms * 1e-3) / 1e9
        # executed bf16 MFMAs of 32x32x16 per 32 rows: 40 per side (initial Grams, three-piece operands),
        # 32 per input head (X^T X), 24 per side (apply)
        exec_flops = (l / 32.0) * (bh * 2 * (40 + 24) + (bh + bkv) * 32) * 2.0 * 32 * 32 * 16
        roof = {"bound": "hbm", "kernel": "pf_sums_kernel + pf_pass_bf16_kernel + pf_xtx_kernel + pf_apply_shared_kernel "
                                          "(two readings of Q, three of K); pf_gramdom_kernel (fp64 d x d algebra per "
                                          "head, latency-bound) between them",
                "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                "traffic": None, "hbm_bytes_per_call": round(bytes_g),
                "algorithmic_flops_per_call": round(flops), "algorithmic_equiv_tflops": round(tf, 2),
                "executed_bf16_mfma_tflops": round(exec_flops / (ms * 1e-3) / 1e12, 1),
                "executed_bf16_mfma_frac": round(exec_flops / (ms * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4),
                "readings_of_the_long_axis": {"Q": 2, "K": 3}, "row_by_row_formulation_readings": 1 + iters}
    elif e == 2 and d <= 128:
        # bf16 input: the passes run on the bf16 matrix cores (fp32 operands as three bf16 pieces), where the
        # arithmetic is far from any limit; what bounds them is the stream over X and A
        gbs = bytes_ / (ms * 1e-3) / 1e9
        # executed bf16 flops: per 32 rows 24 (apply) + 8 (identity) + 24 + 16 (Grams) MFMAs of 32x32x16
        mf_apply, mf_gram = 72, 48
        exec_flops = bh * (l / 32.0) * (2 * mf_gram + iters * 2 * mf_apply) * 2.0 * 32 * 32 * 16
        roof = {"bound": "hbm", "kernel": "pf_pass_bf16_kernel", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                "hbm_bytes_per_call": round(bytes_), "algorithmic_flops_per_call": round(flops),
                "algorithmic_tflops": round(tf, 2),
                "executed_bf16_mfma_tflops": round(exec_flops / (ms * 1e-3) / 1e12, 1),
                "executed_bf16_mfma_frac": round(exec_flops / (ms * 1e-3) / 1e12 / BF16_MFMA_PEAK_TFLOPS, 4)}
    else:
        roof = {"bound": "mfma", "kernel": "pf_pass_mfma_kernel", "achieved": round(tf, 2),
                "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4),
                "traffic": None, "flops_per_call": round(flops), "hbm_bytes_per_call": round(bytes_),
                "hbm_frac": round(bytes_ / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    out = {"metric": "lrqk_prefill_als_ms", "value": round(ms, 3), "unit": "ms", "n_gpus": 1, "steps": steps,
           "warmup": warm, "ms_per_step": round(ms, 3), "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": f"{w.name}@{l}", "heads": [w.num_heads, w.num_kv_heads], "head_dim": d, "r": r,
                      "max_iter": iters, "tol": tol, "input_dtype": "bf16" if e == 2 else "f32"},
           "rel_residual_K": round((num_k / den_k) ** 0.5, 6), "rel_residual_Q": round((num_q / den_q) ** 0.5, 6),
           "roofline": roof,
           "cpu_baseline": cpu}
    return out


def decoder(a):
    """End-to-end greedy decoding: random-init Llama-3-8B-shaped stack, random token ids, LRQK cache in
    every layer (r 32, k 2048, lite 64).  tokens/s = batch * new_tokens / wall time of the decode phase."""
    from lrqk_amd.decoder import LlamaShapeDecoder, DecoderConfig
    cfg = DecoderConfig(layers=a.layers)
    dev = torch.device("cuda:0")
    t0 = time.perf_counter()
    model = LlamaShapeDecoder(cfg, torch.bfloat16, dev, seed=a.seed, context_scale=a.context_scale)
    model.progress = lambda msg: print(msg, file=sys.stderr, flush=True)
    g = torch.Generator(device=dev).manual_seed(a.seed + 1)
    ids = torch.randint(0, cfg.vocab, (a.batch, a.prompt), generator=g, device=dev)
    cache = model.new_cache(r=32, num_active_tokens=2048, lite_tokens=64, max_iter=(2, 2), tol=(1e-2, 1e-2))
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    toks, t_prefill, t_decode, steps = model.generate(ids, a.new_tokens, cache)
    n_dec = a.new_tokens - 1
    tps = a.batch * n_dec / t_decode
    miss = sel = 0
    for li in range(cfg.layers):
        m_, s_, _ = cache.lwattn[li].miss_stats()
        miss += m_
        sel += s_
    # a few more positions with an event pair around every layer's cache path (update + attention): the share of
    # a decoded position that the path takes, the rest being the projections, MLP and lm_head
    model.path_events = []
    tok = toks[:, -1]
    pos = a.prompt + a.new_tokens - 1
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    extra = 8
    for _ in range(extra):
        tok = model.forward(tok[:, None], pos, cache).argmax(-1)
        pos += 1
    torch.cuda.synchronize()
    t_extra = (time.perf_counter() - t0) / extra
    path_us = sum(e0.elapsed_time(e1) for e0, e1 in model.path_events) * 1e3 / len(model.path_events)
    model.path_events = None
    cpu = None
    if a.cpu_steps > 0:
        # the oracle's cache path (factor update, scan, select, diff, gather, attention) of ONE layer at this batch
        # and context, continued from layer 0's state with stand-in q, k, v; everything else a decoded position
        # needs (projections, MLP, lm_head, the other layers) is not in this figure
        import types
        threads, host = host_threads(a)
        torch.set_num_threads(threads)
        eng0 = cache.lwattn[0]
        wl = types.SimpleNamespace(lite_tokens=64, num_active_tokens=2048, groups=cfg.heads // cfg.kv_heads, r=32,
                                   max_iter=(2, 2), tol=(1e-2, 1e-2))
        o, orc = oracle_from_engine(eng0, wl, threads)
        gq = torch.Generator().manual_seed(a.seed + 7)
        qkv = [(torch.randn((a.batch, cfg.heads, 1, cfg.head_dim), generator=gq).bfloat16(),
                torch.randn((a.batch, cfg.kv_heads, 1, cfg.head_dim), generator=gq).bfloat16(),
                torch.randn((a.batch, cfg.kv_heads, 1, cfg.head_dim), generator=gq).bfloat16()) for _ in range(2)]
        Ko, Vo = o.decode(*qkv[0])          # untimed warm-up step
        t0 = time.perf_counter()
        Ko, Vo = o.decode(*qkv[1])
        orc.attention(qkv[1][0], Ko, Vo, torch.float32)
        cpu_s = time.perf_counter() - t0
        cpu = {"value": round(cpu_s * 1e6, 1), "unit": "us/layer-step (cache path only)", "cores": threads, "kind": "port",
               "sample": f"one decode step of layer 0's cache path at batch {a.batch} continued from the GPU state "
                         f"(stand-in q, k, v); compare with cache_path_us_per_layer_step"}
        cpu.update(host)
    out = {"metric": "lrqk_decoder_tokens_per_s", "value": round(tps, 2), "unit": "tokens/s", "n_gpus": 1,
           "steps": n_dec, "warmup": 0, "ms_per_step": round(t_decode / n_dec * 1e3, 3), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": f"llama3_8b_shape_decoder@{a.prompt}", "layers": cfg.layers, "batch": a.batch,
                      "prompt_tokens": a.prompt, "new_tokens": a.new_tokens, "r": 32, "k": 2048, "lite": 64,
                      "context_scale": a.context_scale,
                      "max_iter": [2, 2]},
           "prefill_s": round(t_prefill, 3), "decode_s": round(t_decode, 3), "setup_s": round(setup_s, 2),
           "reference_style_tokens_per_s": round(a.batch * len(steps) / max(sum(steps), 1e-9), 2),
           "us_per_layer_step": round(t_decode / n_dec / cfg.layers * 1e6, 1),
           "last_step_hit_rate": round(1.0 - miss / max(sel, 1), 4),
           "context_scale": a.context_scale,
           "cache_path_us_per_layer_step": round(path_us, 1),
           "other_us_per_layer_step": round(t_extra / cfg.layers * 1e6 - path_us, 1),
           "roofline": None, "cpu_baseline": cpu}
    return out


def host_threads(a):
    """Threads for the CPU legs: every core this process may use (its affinity mask, and the share of the host that
    OMP_NUM_THREADS names where the machine is shared between jobs), with the counts it was chosen from."""
    n_all = os.cpu_count() or 1
    try:
        n_aff = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        n_aff = n_all
    try:
        share = int(os.environ.get("OMP_NUM_THREADS", "0"))
    except ValueError:
        share = 0
    n = a.cpu_threads or max(1, min(n_aff, share or n_aff))
    return n, {"host_cpu_count": n_all, "cpus_in_affinity_mask": n_aff, "omp_num_threads_env": share or None}


def decode_bench(a, compact=False):
    """One decode-mode measurement; returns the result line as a dict (compact: the few keys of a sub-result)."""
    from lrqk_amd import synth
    import lrqk_amd
    from lrqk_amd import ops as ops_mod
    import dataclasses
    dev = torch.device("cuda:0")
    w = synth.WORKLOADS[a.workload]
    if a.seqs > 0 and a.seqs != w.batch:
        w = dataclasses.replace(w, batch=a.seqs)
    if a.max_iter > 0:
        w = dataclasses.replace(w, max_iter=(a.max_iter, a.max_iter), tol=(a.tol, a.tol))
    if a.rank or a.topk or a.lite:
        w = dataclasses.replace(w, r=a.rank or w.r, num_active_tokens=a.topk or w.num_active_tokens,
                                lite_tokens=a.lite or w.lite_tokens)
    if a.data_rank:
        w = dataclasses.replace(w, rho=a.data_rank)
    l = a.context or w.context
    t_setup = time.perf_counter()
    # synthetic prompt, drawn on the GPU (128K x 48 heads x 128 would take minutes on the host)
    Q, K, V, bases, gen = synth.prompt_qkv(w, a.seed, l, device=dev)
    A0 = synth.init_factors(w, l, a.seed + 1, device=dev)
    cls = lrqk_amd.LightAttentionIndicesNoHitMiss if a.variant == "no_hit_miss" else lrqk_amd.LightAttentionIndicesFactory

    def make_engine():
        e_ = cls(num_lite_tokens=w.lite_tokens, attn_topk=w.num_active_tokens, num_key_value_groups=w.groups, r=w.r,
                 max_iter=w.max_iter, tol=w.tol, capacity=4096)
        e_.init_factors = A0
        e_.attn_in_step = not a.no_attn
        e_.fetch_mode = a.fetch
        e_.use_score_index = not a.no_score_index
        e_.use_factor_state = a.factor_state
        if a.victim_rows >= 0:
            e_.victim_rows = a.victim_rows
        return e_
    eng = make_engine()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.prefill(Q, K, V)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    others = []
    for _ in range(max(1, a.rotate) - 1):  # further copies of the same layer state, each with buffers of its own
        o_ = make_engine()
        o_.prefill(Q, K, V)
        others.append(o_)
    del A0
    stream = synth.DecodeStream(w, Q[:, :, -1:], bases, gen)
    n_warm = a.warmup + max(0, a.settle)  # all untimed alike; the line reports both numbers
    copies = 1 + len(others)
    # the timed regions, in this order: exactly --steps steps; a longer one (at least --min-timed steps) when --steps
    # is short; a few steps with every scan launch between events; the first copy alone, back to back
    long_steps = a.min_timed if a.steps < a.min_timed else 0
    ev_steps = max(0, a.event_steps)
    warm_steps = max(0, a.warm_steps) if copies > 1 else 0
    total = n_warm + a.steps + long_steps + ev_steps + warm_steps
    qs, ks, vs = [], [], []
    for _ in range(total):
        q, k, v = stream.next()
        qs.append(q.contiguous()); ks.append(k.contiguous()); vs.append(v.contiguous())
    del Q, K, V
    torch.cuda.empty_cache()
    # reserve so that no step of the timed region allocates or grows a buffer
    for e_ in [eng] + others:
        e_.ws.reserve(w.batch * w.num_heads, l + total + 64, w.num_active_tokens,
                      w.num_active_tokens + w.lite_tokens, w.r, w.head_dim)
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_setup

    for i in range(n_warm):
        eng.decode(qs[i], ks[i], vs[i])
        for o_ in others:
            o_.decode(qs[i], ks[i], vs[i])
        if i % 128 == 127:
            torch.cuda.synchronize()  # (untimed: keeps the launch queue short)
    torch.cuda.synchronize()
    cap_before = (eng._A_K.capacity, eng.KVcpu.capacity)

    # The host enqueues a step in less than half the time the GPU needs for it.  Left alone it runs thousands
    # of launches ahead, and once the runtime's launch queue is full (at about 2000 launches here) every
    # further launch waits in a way that leaves gaps on the GPU.  So the host stays at most 128 layer-steps
    # ahead: it waits for a mark recorded that long ago, which the GPU passed long before, and the GPU never
    # runs dry.  The same marks (one per 32 layer-steps) give the spread of the step time.
    mark_every = max(1, 32 // copies)   # engine iterations between marks
    ahead = max(2, 128 // (mark_every * copies))

    def timed_loop(first, count, engines):
        """count steps of every engine in turn, with no event inside a step: (seconds per layer-step, sorted
        microseconds per layer-step of every mark interval, miss counts of the first engine)."""
        marks, counts = [], []
        torch.cuda.synchronize()
        t_ = time.perf_counter()
        for i in range(first, first + count):
            if (i - first) % mark_every == 0:
                marks.append(torch.cuda.Event(enable_timing=True))
                marks[-1].record()
                if len(marks) > ahead:
                    marks[-1 - ahead].synchronize()
            for j, e_ in enumerate(engines):
                e_.decode(qs[i], ks[i], vs[i])
                if j == 0:
                    counts.append(e_.last_miss_count)
        marks.append(torch.cuda.Event(enable_timing=True))
        marks[-1].record()
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t_) / (count * len(engines))
        spans = []
        for j in range(len(marks) - 1):
            n_it = min(mark_every, count - j * mark_every)
            if n_it > 0:
                spans.append(marks[j].elapsed_time(marks[j + 1]) * 1e3 / (n_it * len(engines)))
        return sec, sorted(spans), counts

    engines = [eng] + others
    pos = n_warm
    eng.ws.select_stats(reset=True)
    eng.ws.victim_stats(reset=True)
    m_first = eng.lite_indices[eng.lite_len] - 1
    sec_k, spans_k, counts_k = timed_loop(pos, a.steps, engines)
    pos += a.steps
    sec_v, spans, counts, n_value = sec_k, spans_k, counts_k, a.steps
    if long_steps:
        eng.ws.select_stats(reset=True)
        eng.ws.victim_stats(reset=True)
        m_first = eng.lite_indices[eng.lite_len] - 1
        sec_v, spans, counts = timed_loop(pos, long_steps, engines)
        pos += long_steps
        n_value = long_steps
    # statistics of the region that `value` comes from
    sel_fast, sel_full = eng.ws.select_stats()
    sel_short, sel_over = eng.ws.select_stats_detail()
    host_rows = eng.ws.victim_stats()
    m_last = eng.lite_indices[eng.lite_len] - 1
    grew = cap_before != (eng._A_K.capacity, eng.KVcpu.capacity)

    def pct(p_):
        return round(spans[min(len(spans) - 1, int(p_ * len(spans)))], 2) if spans else None

    # Kernel time of the scan: a separate pass after the timed regions, every launch of the first copy between two
    # HIP events (a pair delays its step by several microseconds, so none is inside a timed region).
    kern_ms, launches = 0.0, 0
    if ev_steps:
        eng.ws.timing_enable(ev_steps, every=1)
        timed_loop(pos, ev_steps, engines)
        kern_ms, launches = eng.ws.timing_read()
        eng.ws.timing_enable(0)
        pos += ev_steps
    rows_scanned, rows_rescored = eng.ws.scan_stats()
    vic_on = eng.victim_rows_effective > 0 and a.fetch == "direct" and a.variant == "default"

    # the same state stepped back to back: its score index largely stays in the last-level cache
    warm_us = None
    if warm_steps:
        warm_us = timed_loop(pos, warm_steps, [eng])[0] * 1e6
        pos += warm_steps

    n_miss = int(torch.stack(counts).sum())
    n_sel = len(counts) * w.batch * w.num_heads * w.num_active_tokens
    e = 2 if w.dtype == torch.bfloat16 else 4
    row_bytes = 2 * w.head_dim * e
    us_step = sec_v * 1e6
    m_avg = (m_first + m_last) / 2.0
    bh = w.batch * w.num_heads
    scan_bytes = bh * m_avg * w.r * e            # what the reference's scan reads: r values per cached token and head
    n_act = w.num_active_tokens + w.lite_tokens
    step_bytes = (scan_bytes + (0 if a.no_attn else 2 * bh * n_act * w.head_dim * e) + bh * n_act * w.head_dim * e
                  + bh * n_act * w.r * e + 4 * bh * w.r * w.head_dim * e + 3 * bh * w.num_active_tokens * 4
                  + n_miss / n_value * row_bytes)

    read_gbs = copy_gbs = pair_us = pair2_us = None
    sweep = None
    if a.probe_mb > 0:
        read_gbs, copy_gbs = ops_mod.probe_bandwidth(min(a.probe_mb, 1024) << 20, 10, dev)
        # what the same event bracket reads around one and around two kernels that do nothing
        pair_us = ops_mod.probe_event_pair(64, dev)
        pair2_us = ops_mod.probe_event_pair(64, dev, kernels=2)
        if not a.no_probe_sweep:
            table, _ = ops_mod.probe_read_sweep(a.probe_mb << 20, 5, dev)
            best = max(table, key=table.get)
            sweep = {"bytes": a.probe_mb << 20, "best_gbs": round(table[best], 1),
                     "best": {"vectors_in_flight": best[0], "nontemporal": bool(best[1]), "workgroups_per_cu": best[2]},
                     "gbs_by_in_flight_nontemporal_wg_per_cu": {f"{k[0]}/{k[1]}/{k[2]}": round(v, 0)
                                                                for k, v in sorted(table.items())}}
            # the same sweep with launches of the size of one score index (slices of the buffer read in turn, so
            # that no launch finds its slice in the last-level cache): what a launch of the scan's size can reach
            slice_b = (bh * int(m_avg) * w.r) // 16 * 16
            if 0 < slice_b <= (a.probe_mb << 20) // 4:
                t2, _ = ops_mod.probe_read_sweep((a.probe_mb << 20) // slice_b * slice_b, 2, dev, slice_bytes=slice_b)
                b2 = max(t2, key=t2.get)
                sweep["launches_of_index_size"] = {
                    "bytes_per_launch": slice_b, "best_gbs": round(t2[b2], 1), "best_us": round(slice_b / t2[b2] / 1e3, 2),
                    "best": {"vectors_in_flight": b2[0], "nontemporal": bool(b2[1]), "workgroups_per_cu": b2[2]},
                    "gbs_by_in_flight_nontemporal_wg_per_cu": {f"{k[0]}/{k[1]}/{k[2]}": round(v, 0)
                                                               for k, v in sorted(t2.items())}}
    # (between events: the profiler's duration of the same kernel is 2 to 3 us shorter; an empty kernel reads
    # pair_us between the same events, and a second one adds as much again, so the share of the bracket that is
    # not the kernel cannot be taken off by such a calibration)
    kern_us = kern_ms * 1e3 / max(launches, 1)

    sidx_on = (not a.no_score_index) and w.r in (16, 32, 64)
    # Bytes one launch of the scan has to move.  Without the score index: the A_K rows.  With it: the 8-bit copy
    # (r + 2 bytes per row) plus the rows it rescores exactly from A_K (counted by the kernel; last launch) plus
    # the candidate pairs it writes -- fewer bytes than the reference's scan reads, which is the point of it.
    if sidx_on and rows_scanned:
        must_move = bh * m_avg * (w.r + 2) + rows_rescored * w.r * e + 8.0 * rows_rescored
    else:
        must_move = scan_bytes
    achieved = must_move / (kern_us * 1e-6) / 1e9 if launches else 0.0
    tr = MEASURED_TRAFFIC.get((w.name, sidx_on)) \
        if a.context is None and a.variant == "default" and w.batch == 1 else None
    traffic = tr["bytes"] if tr else None

    if a.calib_copy_mb > 0:
        src = torch.empty(a.calib_copy_mb << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    cpu = None
    if a.cpu_steps > 0:
        threads, host = host_threads(a)
        torch.set_num_threads(threads)
        o, orc = oracle_from_engine(eng, w, threads)
        extra = [stream.next() for _ in range(a.cpu_steps + 1)]
        extra = [(q.cpu(), k.cpu(), v.cpu()) for q, k, v in extra]
        q, k, v = extra[0]
        Ko, Vo = o.decode(q, k, v)          # untimed warm-up step
        orc.attention(q, Ko, Vo, torch.float32)
        t0 = time.perf_counter()
        for q, k, v in extra[1:]:
            Ko, Vo = o.decode(q, k, v)
            if not a.no_attn:
                orc.attention(q, Ko, Vo, torch.float32)
        cpu_s = (time.perf_counter() - t0) / a.cpu_steps
        cpu = {"value": round(cpu_s * 1e6, 1), "unit": "us/layer-step", "cores": threads, "kind": "port",
               "sample": f"{a.cpu_steps} decode steps of the same workload continued from the GPU state "
                         f"(fp32 torch-CPU factor update + C scan/sort/diff/gather per head on {threads} threads)"}
        cpu.update(host)

    hit_rate = round(1.0 - n_miss / max(n_sel, 1), 4)
    served = round(1.0 - host_rows / max(n_miss, 1), 4) if vic_on else 0.0
    step_frac = round(step_bytes / (us_step * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
    # achieved = bytes the scan kernel has to move per launch (see must_move above) over its duration, so
    # frac is a fraction of the HBM peak; algorithmic_equiv_gbs prices the same duration at the bytes the
    # reference's scan reads (r values of the storage type per cached token and head), which the score
    # index undercuts; traffic = HBM bytes per launch read from hardware counters (profiles/).
    roof = {"bound": "hbm", "kernel": "score_prefilter_kernel" if sidx_on else "score_filter_kernel",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": round(traffic) if traffic else None,
            "traffic_gbs": round(traffic / (kern_us * 1e-6) / 1e9, 1) if traffic and launches else None,
            "traffic_from": {k_: v_ for k_, v_ in tr.items() if k_ != "bytes"} if tr else None,
            "kernel_us": round(kern_us, 2), "launches": launches,
            "launches_timed_in": "a pass of %d steps after the timed regions" % ev_steps,
            "bytes_per_launch": round(must_move),
            "event_pair_around_empty_kernel_us": round(pair_us, 2) if pair_us is not None else None,
            "event_pair_around_two_empty_kernels_us": round(pair2_us, 2) if pair2_us is not None else None,
            "rows_rescored_per_launch": rows_rescored,
            "algorithmic_bytes_per_launch": round(scan_bytes),
            "algorithmic_equiv_gbs": round(scan_bytes / (kern_us * 1e-6) / 1e9, 1) if launches else None,
            "measured_read_gbs": round(max(read_gbs or 0.0, sweep["best_gbs"] if sweep else 0.0), 1) or None,
            "measured_read_gbs_default_probe": round(read_gbs, 1) if read_gbs else None,
            "measured_copy_gbs": round(copy_gbs, 1) if copy_gbs else None,
            "read_probe_sweep": sweep}
    if compact:
        for k_ in ("traffic_from", "read_probe_sweep", "measured_read_gbs", "measured_read_gbs_default_probe",
                   "measured_copy_gbs", "event_pair_around_empty_kernel_us", "event_pair_around_two_empty_kernels_us",
                   "traffic", "traffic_gbs", "launches_timed_in"):
            roof.pop(k_, None)
        return {"workload": f"{w.name}@{l}", "batch": w.batch, "layer_copies": copies, "steps": n_value,
                "us_per_layer_step": round(us_step, 2), "us_per_sequence_layer_step": round(us_step / w.batch, 2),
                "tokens_per_s_32_layers": round(w.batch * 1e6 / (32 * us_step), 2),
                "step_algorithmic_bytes": round(step_bytes), "step_hbm_frac": step_frac,
                "hit_rate": hit_rate, "victim_cache_served": served,
                "h2d_bytes_per_step": round((host_rows if vic_on else n_miss) / n_value * row_bytes),
                "roofline": roof, "cpu_baseline": cpu}

    out = {
        "metric": "lrqk_decode_us_per_layer_step", "value": round(us_step, 2), "unit": "us",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "settle_steps": max(0, a.settle),
        "ms_per_step": round(us_step / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": f"{w.name}@{l}", "batch": w.batch, "heads": [w.num_heads, w.num_kv_heads],
                   "head_dim": w.head_dim, "r": w.r, "k": w.num_active_tokens, "lite": w.lite_tokens, "max_iter": list(w.max_iter),
                   "variant": a.variant, "fetch": a.fetch, "score_index": sidx_on, "attention_in_step": not a.no_attn, "candidates_m": [m_first, m_last],
                   "factor_update": "fp64 from kept state" if a.factor_state else "fp32 over the active rows",
                   "layer_copies": copies,
                   "cache": "cold: %d copies of the layer state take turns, as the layers of a decoder do" % copies
                   if copies > 1 else "warm: one copy stepped back to back"},
        # `value` is timed over value_timed_steps steps of every copy (at least --min-timed: a region of --steps 20
        # lasts 7 ms); the region of exactly --steps steps ran first and is reported beside it
        "value_timed_steps": n_value, "value_timed_layer_steps": n_value * copies,
        "us_per_step_over_exactly_steps": round(sec_k * 1e6, 2),
        "us_per_step_p10_p50_p90": [pct(0.1), pct(0.5), pct(0.9)],
        "us_per_step_one_copy_back_to_back": round(warm_us, 2) if warm_us else None,
        "us_per_sequence_layer_step": round(us_step / w.batch, 2),
        "tokens_per_s_32_layers": round(w.batch * 1e6 / (32 * us_step), 2),
        "hit_rate": hit_rate,
        "h2d_bytes_per_step": round((host_rows if vic_on else n_miss) / n_value * row_bytes),
        "missed_bytes_per_step": round(n_miss / n_value * row_bytes),
        "victim_cache": {"rows_per_head": eng.victim_rows_effective
                         if vic_on else 0,
                         "served": served},
        "step_algorithmic_bytes": round(step_bytes),
        "step_hbm_frac": step_frac,
        "roofline": roof,
        "selector_heads": {"from_candidate_list": sel_fast, "rescanned": sel_full, "list_short": sel_short,
                           "list_overflow": sel_over},
        "cpu_baseline": cpu,
        "prefill_s": round(prefill_s, 3), "setup_s": round(setup_s, 2), "buffers_grew_in_timed_region": grew,
    }
    return out


def also_results(a, t_start):
    """The other configurations, compact, for the `also` key of the default line: 32K decode, four sequences stepped
    together at 128K, the prefill factorisation, the full decoder.  Each runs after the one before it has freed its
    buffers; one that fails leaves its error text in place of a result."""
    import copy
    import gc

    def run(name, fn):
        gc.collect()
        torch.cuda.empty_cache()
        if hasattr(torch._C, "_host_emptyCache"):
            torch._C._host_emptyCache()  # pinned blocks of the earlier stores (the allocator keeps them otherwise)
        free_b, total_b = torch.cuda.mem_get_info()
        print(f"also.{name}: starts with {free_b / 2**30:.1f} of {total_b / 2**30:.1f} GiB of device memory free",
              file=sys.stderr, flush=True)
        t0 = time.perf_counter()
        try:
            res = fn()
        except Exception as ex:  # the main line is still worth printing
            import traceback
            where = [f"{f.name}:{f.lineno}" for f in traceback.extract_tb(ex.__traceback__)[-4:]]
            res = {"error": f"{type(ex).__name__}: {str(ex).splitlines()[0] if str(ex) else ''}", "at": where}
        res["wall_s"] = round(time.perf_counter() - t0, 1)
        print(f"also.{name}: {res['wall_s']} s", file=sys.stderr, flush=True)
        return res

    def sub(**kw):
        b = copy.copy(a)
        b.context, b.seqs, b.probe_mb, b.calib_copy_mb, b.warm_steps = None, 0, 0, 0, 0
        for k_, v_ in kw.items():
            setattr(b, k_, v_)
        return b

    out = {}
    # 32K: eight copies take turns (four copies of its 36 MB index would all stay in the 256 MB last-level cache)
    out["ctx32k"] = run("ctx32k", lambda: decode_bench(
        sub(workload="llama8b_32k_bf16", steps=256, min_timed=256, warmup=16, settle=64, rotate=8, event_steps=32,
            cpu_steps=min(a.cpu_steps, 32)), compact=True))
    out["seqs4"] = run("seqs4", lambda: decode_bench(
        sub(workload="llama8b_128k_bf16", seqs=4, steps=128, min_timed=128, warmup=16, settle=64, rotate=2,
            event_steps=32, cpu_steps=min(a.cpu_steps, 8)), compact=True))

    def pf():
        r_ = prefill_als(sub(workload="llama8b_32k_prefill_als", steps=8, warmup=2, cpu_steps=min(a.cpu_steps, 1)))
        roof = r_["roofline"]
        return {"workload": r_["config"]["workload"], "ms": r_["value"], "rel_residual_K": r_["rel_residual_K"],
                "rel_residual_Q": r_["rel_residual_Q"], "max_iter": r_["config"]["max_iter"],
                "roofline": {k_: roof.get(k_) for k_ in ("bound", "achieved", "peak", "unit", "frac", "hbm_bytes_per_call",
                                                          "executed_bf16_mfma_tflops", "executed_bf16_mfma_frac",
                                                          "readings_of_the_long_axis")},
                "cpu_baseline": r_["cpu_baseline"]}
    out["prefill_als"] = run("prefill_als", pf)

    if a.also_decoder and time.perf_counter() - t_start < a.also_budget_s:
        def dec():
            r_ = decoder(sub(layers=32, batch=4, prompt=65536, new_tokens=128, context_scale=5.0,
                             cpu_steps=min(a.cpu_steps, 1)))
            keep = ("value", "unit", "prefill_s", "decode_s", "us_per_layer_step", "last_step_hit_rate",
                    "cache_path_us_per_layer_step", "other_us_per_layer_step", "cpu_baseline")
            res = {k_: r_[k_] for k_ in keep}
            res["workload"] = r_["config"]["workload"] + " x 4 sequences, 32 layers, 128 new tokens, context_scale 5"
            return res
        out["decoder"] = run("decoder", dec)
    else:
        out["decoder"] = {"skipped": "off (--no-also-decoder)" if not a.also_decoder else
                          "the run had already taken %.0f s" % (time.perf_counter() - t_start)}
    return out


def main():
    t_start = time.perf_counter()
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: the LRQK cache path has no multi-GPU part (heads shard trivially); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    from lrqk_amd import _lib
    _lib.load()  # fail loudly if the HIP library is missing
    if a.mode == "prefill_als":
        print(json.dumps(prefill_als(a)))
        return
    if a.mode == "decoder":
        print(json.dumps(decoder(a)))
        return
    out = decode_bench(a)
    plain = (a.workload == "llama8b_128k_bf16" and a.context is None and a.variant == "default" and not a.seqs
             and not (a.rank or a.topk or a.lite or a.max_iter or a.data_rank) and not a.no_attn)
    if a.also == "on" or (a.also == "auto" and plain):
        out["also"] = also_results(a, t_start)
    out["wall_s"] = round(time.perf_counter() - t_start, 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
