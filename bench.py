#!/usr/bin/env python3
"""Decode benchmark: tokens/s of the batch-1 KV-cache greedy token loop on one MI355X.

A "step" is one decoded token (one pass of the whole token loop: embedding row, every layer,
final norm, tied LM head, argmax).  The default workload is the configuration the headline metric
is quoted on: the 600M-class bf16 model (dim 1536, 24 layers, 12 heads x 128, hidden 4096, vocab
32768, seq 2048), a 128-token random prompt, greedy decode at batch 1.  Weights are synthetic
N(0, 0.02) from a fixed seed and already resident in HBM when the timed region starts.

Prints ONE JSON line (see the keys below).  `roofline.achieved` is the algorithmic bytes one token
step streams (weights + scales + norms + one embedding row + the KV rows it reads and writes) divided
by the per-step device time measured with HIP events on the model's own stream.
`cpu_baseline` times the CPU oracle's cached token loop on a bounded number of steps of the same
model on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

HBM_PEAK_GBPS = 8000.0

WORKLOADS = {
    # name: (config factory name, weight dtype, kv dtype, prompt tokens, generated steps)
    "c1_tiny_fp32": ("config_c1", "F32", "F32", 4, 32),
    "c2_600m_bf16_bs1": ("config_600m", "BF16", "BF16", 128, 256),
    "c4_5b_bf16_bs1": ("config_5b", "BF16", "BF16", 1024, 128),
    "c5_5b_fp8_bs1": ("config_5b", "FP8_E4M3", "BF16", 512, 256),
    "c5_5b_int4_bs1": ("config_5b", "INT4_G128", "BF16", 512, 256),
    # 8 samples over one shared 512-token prompt, temperature 0.8, top-k 8, stepped together
    "c3_600m_bf16_8samples": ("config_600m", "BF16", "BF16", 512, 256),
    # the same request on the 5B model with 4-bit / 8-bit weights (the multi-sample step as one kernel per product)
    "c5_5b_int4_8samples": ("config_5b", "INT4_G128", "BF16", 512, 128),
    "c5_5b_fp8_8samples": ("config_5b", "FP8_E4M3", "BF16", 512, 128),
}
MULTI_SAMPLE_WORKLOADS = ("c3_600m_bf16_8samples", "c5_5b_int4_8samples", "c5_5b_fp8_8samples")
C3_SAMPLES, C3_TEMPERATURE, C3_TOP_K = 8, 0.8, 8
ALL_CONFIG_ORDER = ["c1_tiny_fp32", "c2_600m_bf16_bs1", "c3_600m_bf16_8samples", "c4_5b_bf16_bs1", "c5_5b_fp8_bs1",
                    "c5_5b_int4_bs1", "c5_5b_int4_8samples", "c5_5b_fp8_8samples"]
# timed steps of the short runs behind the all_configs entries (generated steps - 1 of the workload, capped)
ALL_CONFIG_STEPS = {"c1_tiny_fp32": 31, "c2_600m_bf16_bs1": 255, "c3_600m_bf16_8samples": 64, "c4_5b_bf16_bs1": 32,
                    "c5_5b_fp8_bs1": 64, "c5_5b_int4_bs1": 64, "c5_5b_int4_8samples": 32, "c5_5b_fp8_8samples": 32}

# HBM bytes per launch of the dominant kernel from hardware counters (FETCH_SIZE + WRITE_SIZE, each
# scaled by what the same counter reads for a plain copy of known size): measured separately with
# rocprofv3 --pmc and recorded in profiles/k_lean_c2_600m_bf16_bs1.md, profiles/k_mega_hbm_traffic_c1_c4_c5.md and
# profiles/k_rows_c3_600m_bf16_8samples.md
# (per step, i.e. the LM-head GEMV included where it is a launch of its own, at the KV length of the
# profiled run); a benchmark run cannot collect it itself.
TRAFFIC_SOURCE = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries under profiles/, not measured in this run"
MEASURED_TRAFFIC_BYTES = {"c1_tiny_fp32": 1.267e8, "c2_600m_bf16_bs1": 1.5092e9, "c3_600m_bf16_8samples": 1.811e9,
                          "c4_5b_bf16_bs1": 1.3874e10, "c5_5b_fp8_bs1": 7.118e9, "c5_5b_int4_bs1": 4.008e9}


def run_c3(args, workload, cfg, weights, n_prompt, wdt, kvdt):
    """Multi-sample workload through the session layer: a step is one pass of the weights that
    advances all 8 samples by one token (per-block top-k candidates, their merge and the reference's
    draw, all on the device: the whole request is one enqueued run); value = sampled tokens per
    second over all samples."""
    from rustane_amd import engine as E
    from rustane_amd import synth
    prompt = synth.make_prompt(7, cfg.vocab, n_prompt)
    s = E.InferenceSession(cfg, weights, prompt, weight_dtype=int(wdt), kv_dtype=int(kvdt))
    K, W = args.steps, args.warmup
    room = cfg.seq - n_prompt - 1
    K = min(K, room)

    def request(steps, seed):
        return E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=steps + 1, temperature=C3_TEMPERATURE,
                                   top_k=C3_TOP_K, samples=C3_SAMPLES, seed=seed)
    if W > 0:
        s.generate(request(min(W, room), args.seed))
    t0 = time.perf_counter()
    got = s.generate(request(K, args.seed))
    wall = time.perf_counter() - t0
    dev_ms = s.batch_device_ms()
    decode_s = got.total_decode_elapsed
    mean_kv = n_prompt + (K + 1) // 2
    w_bytes = s.bytes_per_token(0)
    bytes_per_step = w_bytes + C3_SAMPLES * (s.bytes_per_token(mean_kv) - w_bytes)
    achieved = bytes_per_step * K / (dev_ms * 1e-3) / 1e9
    flops_per_step = 2.0 * C3_SAMPLES * cfg.param_count()              # every weight multiplies every row once
    return {
        "metric": "decode tok/s @600M bf16 bs1; % of HBM peak GB/s; prefill ms",
        "value": C3_SAMPLES * K / decode_s, "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": decode_s * 1e3 / K, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"F32": "f32", "BF16": "bf16", "FP8_E4M3": "fp8_e4m3", "INT4_G128": "int4"}[wdt.name], "data": "synthetic",
        "config": {"workload": workload, "prompt_tokens": n_prompt, "batch": C3_SAMPLES, "kv_dtype": kvdt.name.lower(),
                   "temperature": C3_TEMPERATURE, "top_k": C3_TOP_K, "params": cfg.param_count(), "mean_kv_len": mean_kv},
        "prefill_ms": s.prefill_elapsed() * 1e3, "request_wall_ms": wall * 1e3,
        "device_ms_per_step": dev_ms / K,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get(workload),
                     "traffic_source": TRAFFIC_SOURCE, "bytes_per_step": bytes_per_step},
        "mfma_roofline": {"bound": "mfma", "achieved": flops_per_step * K / (dev_ms * 1e-3) / 1e12, "peak": 2500.0,
                          "unit": "TFLOP/s", "frac": flops_per_step * K / (dev_ms * 1e-3) / 2.5e15},
        "sampled_head": [int(r.sampled[1]) for r in got.results],
    }


def cpu_baseline(cfg, weights, kv_bf16, prompt=None, gpu_stream=None, budget_s=20.0, max_steps=64, naive_steps=-1):
    """Times the oracle's KV-cached greedy loop (the CPU restatement of the reference's arithmetic) on
    this box's host cores.  With a prompt (the small workloads) the oracle replays the workload itself
    -- window forward over the prompt, then greedy steps -- and its tokens are compared with the
    GPU's stream; otherwise it steps from an empty cache (the weight stream dominates the cost, so the
    rate barely depends on the position).  Returns the cpu_baseline object."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    orc = O.Oracle(cfg, weights, kv_round_bf16=kv_bf16)
    extra, tok = {}, 1
    if prompt is not None:
        lg, _, _ = orc.forward_window(prompt)
        tok = int(O.argmax_last(lg[0]))
        cpu_stream = [tok]
    n, t0 = 0, time.perf_counter()
    while n < max_steps and orc.len() < cfg.seq:
        lg = orc.decode_logits_from_id(tok)
        tok = int(O.argmax_lower(lg))
        n += 1
        if prompt is not None:
            cpu_stream.append(tok)
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    if prompt is not None and gpu_stream is not None:
        m = min(len(cpu_stream), len(gpu_stream))
        div = next((i for i in range(m) if cpu_stream[i] != int(gpu_stream[i])), None)
        extra = {"greedy_tokens_compared": m, "first_divergence_step": div}
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    what = "after the workload's prompt" if prompt is not None else "from an empty cache"
    out = {"value": n / dt, "unit": "tok/s", "cores": cores, "kind": "port",
           "sample": "%d KV-cached greedy steps of the same model %s, fp32 CPU oracle" % (n, what)}
    out.update(extra)
    steps = 0
    if prompt is not None:
        # the reference's other decode mode on the same cores: every token is a forward pass over the whole
        # cfg.seq window from position 0 (crates/engine/src/inference.rs:650-700).  All 32 steps of the tiny
        # workload, one of the 600M one (~3 TFLOP: 13 s on the 16 host cores of the GPU box) unless --cpu-naive-steps
        # says otherwise.
        steps = naive_steps if naive_steps >= 0 else (32 if cfg.nlayers * cfg.dim <= 8192 else 1)
    if prompt is not None and steps > 0:
        window = np.resize(np.asarray(prompt, np.uint32), cfg.seq)
        naive = O.Oracle(cfg, weights, kv_round_bf16=kv_bf16)
        t1 = time.perf_counter()
        for _ in range(steps):
            naive.forward_window(window)
        dn = time.perf_counter() - t1
        out["naive_full_context"] = {"value": steps / dn, "unit": "tok/s",
                                     "sample": "%d whole-window (%d positions) forward passes of the same oracle" % (steps, cfg.seq)}
    return out


def run_c4_sampled(args, workload, cfg, dev, kvdt, prompt_logits, n_prompt, gen_steps, prefill_dev_ms, prefill_wall_ms,
                   prefill_flops, mfma_peak):
    """The 5B workload as defined: full-vocabulary sampling at temperature 1.0 through the exact
    block-stats path (crates/engine/src/inference.rs:600-625) -- per token one decode step that
    leaves per-block (max, sum exp) on the device, a block drawn from them, the token drawn inside
    that block's logits (two uniforms per token, the reference's LCG, seed 1).  Both draws run on the
    device with the host's arithmetic, so the K steps are one enqueued run."""
    import ctypes as C
    from rustane_amd import engine as E
    L = E.lib()
    fp = C.POINTER(C.c_float)
    rng = C.c_uint64(1)
    T = 1.0
    lg = np.ascontiguousarray(prompt_logits, np.float32)
    cur = int(L.rs_sample_next(lg.ctypes.data_as(fp), lg.size, T, 0, C.byref(rng)))
    K, W = args.steps, args.warmup
    K = min(K, gen_steps - 1, cfg.seq - n_prompt - W - 1)

    state = rng.value
    if W > 0:
        toks, state = dev.decode_fullvocab_sampled_run(cur, T, state, W)
        cur = int(toks[-1])
    kv0 = dev.len()
    t0 = time.perf_counter()
    toks, state = dev.decode_fullvocab_sampled_run(cur, T, state, K)
    wall = time.perf_counter() - t0
    dev_ms = dev.last_device_ms()
    mean_kv = kv0 + (K + 1) // 2
    bytes_per_step = dev.bytes_per_token(mean_kv)
    achieved = bytes_per_step * K / (dev_ms * 1e-3) / 1e9
    return {
        "metric": "decode tok/s @600M bf16 bs1; % of HBM peak GB/s; prefill ms",
        "value": K / wall, "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": wall * 1e3 / K,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": workload, "prompt_tokens": n_prompt, "batch": 1, "kv_dtype": kvdt.name.lower(),
                   "sampler": "full-vocab block stats, temperature 1.0", "params": cfg.param_count(), "mean_kv_len": mean_kv},
        "prefill_ms": prefill_dev_ms, "prefill_wall_ms": prefill_wall_ms,
        "prefill_roofline": {"bound": "mfma", "achieved": prefill_flops / (prefill_dev_ms * 1e-3) / 1e12,
                             "peak": mfma_peak / 1e12, "unit": "TFLOP/s",
                             "frac": prefill_flops / (prefill_dev_ms * 1e-3) / mfma_peak},
        "device_ms_per_step": dev_ms / K,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get(workload),
                     "traffic_source": TRAFFIC_SOURCE, "bytes_per_step": bytes_per_step},
        "sampled_head": [int(t) for t in toks[:4]],
    }


def per_call_paths(dev, cfg, first, n_prompt, steps, chained_ms):
    """The three per-token shapes the reference's own decode micro-benchmarks time
    (crates/engine/tests/bench_decode_input_path.rs:132-235), each `steps` SYNCHRONOUS calls through the
    C ABI from the end of the prompt: greedy argmax from the token id; per-block top-k candidates (k = 8, the
    host merge and draw of the reference's loop included); block statistics, the host's block draw, the
    block's logits and the host's token draw (temperature 0.8).  ms per token, wall clock, preallocated
    buffers, the calls made straight through ctypes."""
    import ctypes as C
    from rustane_amd import engine as E
    lib, eng, h = dev._lib, E.lib(), dev._h
    fp, up = C.POINTER(C.c_float), C.POINTER(C.c_uint32)
    B, K8, T = dev.blocks, 8, 0.8
    out = {"steps": steps, "chained_device_ms_per_step": chained_ms}
    tok = C.c_uint32()

    def timed(body):
        dev.set_len(n_prompt)
        body(2)                                   # the variant's graph is captured on its first call
        dev.set_len(n_prompt)
        t0 = time.perf_counter()
        body(steps)
        return (time.perf_counter() - t0) * 1e3 / steps

    def greedy(n):
        cur = first
        for _ in range(n):
            rc = lib.hipdec_decode_token_argmax_from_id(h, cur, C.byref(tok))
            assert rc == 0, rc
            cur = tok.value
    out["argmax_from_id_ms"] = timed(greedy)

    vals, idxs = np.empty(B * K8, np.float32), np.empty(B * K8, np.uint32)
    mv, mi = np.empty(K8, np.float32), np.empty(K8, np.uint32)
    cnt, rng = C.c_size_t(), C.c_uint64(1)
    vp, ip, mvp, mip = vals.ctypes.data_as(fp), idxs.ctypes.data_as(up), mv.ctypes.data_as(fp), mi.ctypes.data_as(up)
    eng.rs_merge_topk_candidates.restype = C.c_uint64
    eng.rs_merge_topk_candidates.argtypes = [fp, up, C.c_size_t, C.c_size_t, fp, up]
    eng.rs_sample_topk_candidates.restype = C.c_uint32
    eng.rs_sample_topk_candidates.argtypes = [up, fp, C.c_size_t, C.c_float, C.POINTER(C.c_uint64)]

    def topk(n):
        cur = first
        for _ in range(n):
            rc = lib.hipdec_decode_token_topk_from_id(h, cur, K8, vp, ip, B * K8, C.byref(cnt))
            assert rc == 0, rc
            m = eng.rs_merge_topk_candidates(vp, ip, cnt.value, K8, mvp, mip)
            cur = eng.rs_sample_topk_candidates(mip, mvp, m, T, C.byref(rng))
    out["topk8_candidates_from_id_ms"] = timed(topk)

    mx, sm, blk = np.empty(B, np.float32), np.empty(B, np.float32), np.empty(256, np.float32)
    mxp, smp, bp = mx.ctypes.data_as(fp), sm.ctypes.data_as(fp), blk.ctypes.data_as(fp)
    valid = C.c_size_t()
    eng.rs_sample_block_from_stats.restype = C.c_uint64
    eng.rs_sample_block_from_stats.argtypes = [fp, fp, C.c_size_t, C.POINTER(C.c_uint64)]
    eng.rs_sample_block_logits.restype = C.c_uint32
    eng.rs_sample_block_logits.argtypes = [C.c_uint32, fp, C.c_size_t, C.c_float, C.POINTER(C.c_uint64)]
    inv_t = float(np.float32(1.0) / np.float32(T))

    def stats(n):
        cur = first
        for _ in range(n):
            rc = lib.hipdec_decode_token_block_stats_from_id(h, cur, C.c_float(inv_t), C.c_float(0.0), mxp, smp, B, C.byref(cnt))
            assert rc == 0, rc
            b = eng.rs_sample_block_from_stats(mxp, smp, cnt.value, C.byref(rng))
            rc = lib.hipdec_materialize_current_logits_block(h, b, C.c_float(0.0), bp, 256, C.byref(valid))
            assert rc == 0, rc
            cur = eng.rs_sample_block_logits(b * 256, bp, valid.value, T, C.byref(rng))
    out["block_stats_then_block_from_id_ms"] = timed(stats)
    dev.set_len(n_prompt)
    return out


_WEIGHTS = {}


def cached_weights(cfg_name, cfg, seed, round_bf16):
    """Synthetic N(0, 0.02) weights of a configuration; the latest set is kept, since consecutive
    workloads share their model (the 5B fp32 master copy is 26 GB of host memory)."""
    from rustane_amd import synth
    key = (cfg_name, seed, round_bf16)
    if key not in _WEIGHTS:
        _WEIGHTS.clear()
        _WEIGHTS[key] = synth.make_weights(cfg, seed=seed, std=0.02, round_bf16=round_bf16)
    return _WEIGHTS[key]


def measure(args, workload, with_cpu_baseline):
    """One workload, start to finish: weights, prefill (reported), the timed decode region; returns the
    result object (the keys of the benchmark line)."""
    from rustane_amd import synth
    from rustane_amd.hipdec import HipDecodeModel, KvDtype, WeightDtype

    cfg_name, wdt, kvdt, n_prompt, gen_steps = WORKLOADS[workload]
    cfg = getattr(synth, cfg_name)()
    wdt, kvdt = WeightDtype[wdt], KvDtype[kvdt]
    weights = cached_weights(cfg_name, cfg, args.seed, wdt != WeightDtype.F32)
    if workload in MULTI_SAMPLE_WORKLOADS:
        return run_c3(args, workload, cfg, weights, n_prompt, wdt, kvdt)
    dev = HipDecodeModel(cfg, weights, weight_dtype=wdt, kv_dtype=kvdt)
    prompt = synth.make_prompt(7, cfg.vocab, n_prompt)

    # prefill (reported, not part of the timed decode region): one untimed pass that also allocates
    # the prefill workspace, then the measured pass from an empty cache
    dev.prefill(prompt)
    dev.set_len(0)
    t0 = time.perf_counter()
    logits = dev.prefill(prompt)
    prefill_wall_ms = (time.perf_counter() - t0) * 1e3
    prefill_dev_ms = dev.last_device_ms()
    first = int(np.argmax(logits))
    # The same prompt under the other activation formats of the prefill GEMMs (the headline figure is the
    # model's default: one fp16 number per activation for 8-bit / 4-bit weights with a bf16 cache, the (hi, lo)
    # bf16 pair otherwise); differences are against the default's prompt logits.  The cache is rebuilt with the default afterwards.
    prefill_options = None
    if wdt != WeightDtype.F32 and n_prompt > 32:
        default_mode = 2 if (kvdt == KvDtype.BF16 and wdt in (WeightDtype.FP8_E4M3, WeightDtype.INT4_G128)) else 0
        prefill_options = {"default": ("bf16_pair", "bf16", "f16")[default_mode] + "_activations"}
        # (mixed: the pair into the q/k/v and output projections, single bf16 numbers into the two feed-forward products)
        for name, mode in (("bf16_pair_activations", 0), ("bf16_activations", 1), ("f16_activations", 2), ("mixed_pair_attention_bf16_ffn", 3)):
            if mode == default_mode:
                continue
            dev.set_prefill_activations(mode)
            dev.set_len(0)
            lg1 = dev.prefill(prompt)
            prefill_options[name] = {"prefill_ms": dev.last_device_ms(),
                                     "max_logit_diff_rel": float(np.abs(lg1 - logits).max() / np.abs(logits).max()),
                                     "same_first_token": bool(int(np.argmax(lg1)) == first)}
        dev.set_prefill_activations(default_mode)
        dev.set_len(0)
        dev.prefill(prompt)
    # algorithmic prefill flops: 2*T*(linear params) + causal attention + the LM head on the last row
    lin = cfg.nlayers * (cfg.dim * (cfg.q_dim + 2 * cfg.kv_dim) + cfg.q_dim * cfg.dim + 3 * cfg.dim * cfg.hidden)
    T = n_prompt
    prefill_flops = 2.0 * T * lin + cfg.nlayers * 4.0 * cfg.heads * cfg.hd * T * (T + 1) / 2 + 2.0 * cfg.vocab * cfg.dim
    mfma_peak = {"F32": 157.3e12, "BF16": 2.5e15, "FP8_E4M3": 2.5e15, "INT4_G128": 2.5e15}[wdt.name]

    room = cfg.seq - n_prompt
    K, W = args.steps, args.warmup
    if workload == "c4_5b_bf16_bs1":
        out = run_c4_sampled(args, workload, cfg, dev, kvdt, logits, n_prompt, gen_steps, prefill_dev_ms, prefill_wall_ms,
                             prefill_flops, mfma_peak)
        out["prefill_options"] = prefill_options
        return out
    if W > 0:
        dev.decode_greedy_run(first, min(W, room))
    # timed region: exactly K greedy steps, in runs that restart at the end of the prompt so every
    # run sees the same KV lengths the workload defines; each run call returns after a stream sync
    run_len = min(gen_steps - 1, room)
    done, wall, dev_ms, kv_sum = 0, 0.0, 0.0, 0
    while done < K:
        n = min(run_len, K - done)
        dev.set_len(n_prompt)
        t0 = time.perf_counter()
        run = dev.decode_greedy_run(first, n)
        wall += time.perf_counter() - t0
        if done == 0:
            gpu_stream = [first] + [int(t) for t in run]
        dev_ms += dev.last_device_ms()
        kv_sum += sum(range(n_prompt + 1, n_prompt + n + 1))
        done += n
    if args.calibrate_copy:
        from rustane_amd.hipdec import calibration_copy
        calibration_copy(args.calibrate_copy << 20, 4)
    mean_kv = kv_sum // max(done, 1)
    bytes_per_step = dev.bytes_per_token(mean_kv)
    achieved = bytes_per_step * K / (dev_ms * 1e-3) / 1e9

    out = {
        "metric": "decode tok/s @600M bf16 bs1; % of HBM peak GB/s; prefill ms",
        "value": K / wall,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": wall * 1e3 / K,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"F32": "f32", "BF16": "bf16", "FP8_E4M3": "fp8_e4m3", "INT4_G128": "int4"}[wdt.name],
        "data": "synthetic",
        "config": {"workload": workload, "prompt_tokens": n_prompt, "batch": 1, "kv_dtype": kvdt.name.lower(),
                   "params": cfg.param_count(), "mean_kv_len": mean_kv},
        "prefill_ms": prefill_dev_ms,
        "prefill_wall_ms": prefill_wall_ms,
        "prefill_roofline": {"bound": "mfma", "achieved": prefill_flops / (prefill_dev_ms * 1e-3) / 1e12,
                             "peak": mfma_peak / 1e12, "unit": "TFLOP/s",
                             "frac": prefill_flops / (prefill_dev_ms * 1e-3) / mfma_peak},
        "device_ms_per_step": dev_ms / K,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get(workload),
                     "traffic_source": TRAFFIC_SOURCE, "bytes_per_step": bytes_per_step},
    }
    if prefill_options:
        out["prefill_options"] = prefill_options
    if workload == "c2_600m_bf16_bs1" and not args.no_per_call:
        out["per_call"] = per_call_paths(dev, cfg, first, n_prompt, 48, dev_ms / K)
    if with_cpu_baseline:
        replay = workload in ("c1_tiny_fp32", "c2_600m_bf16_bs1")      # the oracle can afford the prompt here
        out["cpu_baseline"] = cpu_baseline(cfg, weights, kvdt == KvDtype.BF16, prompt if replay else None,
                                           gpu_stream if replay else None, naive_steps=args.cpu_naive_steps)
    return out


def summary(r):
    """What the all_configs entry of the benchmark line keeps of a workload's result."""
    e = {"dtype": r["dtype"], "kv_dtype": r["config"]["kv_dtype"], "batch": r["config"]["batch"],
         "prompt_tokens": r["config"]["prompt_tokens"], "steps": r["steps"], "tok_s": r["value"],
         "ms_per_step": r["ms_per_step"], "device_ms_per_step": r["device_ms_per_step"], "prefill_ms": r["prefill_ms"],
         "roofline_frac": r["roofline"]["frac"], "achieved_GBps": r["roofline"]["achieved"],
         "bytes_per_step": r["roofline"]["bytes_per_step"]}
    if "prefill_roofline" in r:
        e["prefill_mfma_frac"] = r["prefill_roofline"]["frac"]
    if r.get("prefill_options"):
        e["prefill_options"] = r["prefill_options"]
    if "mfma_roofline" in r:
        e["step_mfma_frac"] = r["mfma_roofline"]["frac"]
    if "per_call" in r:
        e["per_call"] = r["per_call"]
    if "cpu_baseline" in r:
        e["cpu_baseline"] = r["cpu_baseline"]
    return e


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=255)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--workload", default="c2_600m_bf16_bs1", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-call", action="store_true",
                    help="skip the synchronous call-per-token figures of the 600M workload")
    ap.add_argument("--no-all-configs", action="store_true",
                    help="only the selected workload (by default the line also carries a short run of every other one)")
    ap.add_argument("--cpu-naive-steps", type=int, default=-1, metavar="N",
                    help="whole-window forward passes of the CPU oracle to time beside its KV-cached loop "
                         "(default: 32 for the tiny workload, 1 for the 600M one)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="also run 4 launches of a plain copy kernel of this size (for scaling traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this decode path runs on one GPU (no sharding); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    out = measure(args, args.workload, not args.no_cpu_baseline)
    if not args.no_all_configs:
        # the other workloads of the benchmark definition, each over its own prompt and a bounded
        # number of steps, in the same process (their full-length runs: --workload NAME)
        allc = {args.workload: summary(out)}
        short = argparse.Namespace(**vars(args))
        short.calibrate_copy = 0
        for name in ALL_CONFIG_ORDER:
            if name == args.workload:
                continue
            short.steps, short.warmup = ALL_CONFIG_STEPS[name], 4
            # (the tiny workload is the one the CPU can replay whole: its entry carries the CPU figures of both decode modes)
            allc[name] = summary(measure(short, name, name == "c1_tiny_fp32" and not args.no_cpu_baseline))
        out["all_configs"] = allc
    print(json.dumps(out))


if __name__ == "__main__":
    main()
