#!/usr/bin/env python3
"""Writes the full-size known-answer vectors under tests/golden/ with the CPU oracle.

The reference holds no golden files for the decode path (its parity tests compare two of its own
backends at run time, crates/engine/tests/auto_kv_decode.rs), so these vectors are the CPU oracle's
answers on the benchmark workloads, computed once where CPU time is cheap: the 600M-class model
(dim 1536, 24 layers, 12 heads x 128, hidden 4096, vocab 32768) with bf16-rounded synthetic weights
and the 128-token benchmark prompt, then greedy decoding.  Two cases: weight scale 0.02 with a bf16
KV cache (the benchmark's own definition; its greedy stream soon repeats one token), and weight
scale 0.05 with an fp32 KV cache (the stream keeps moving; with a bf16 cache a 1-ulp difference in a
cached value flips its rounding and a stream this sensitive is not a stable known answer).

Each vector holds the 32 largest prompt logits (index, value), the whole-vocabulary logit checksum
and the greedy stream over the workload's 256 steps, with the smallest gap between the two largest
logits met on the way (a stream is a usable known answer only while that gap stays far above the
logit tolerance); the fp32-cache case also holds two sampled streams of the reference's cached
loop (crates/engine/src/inference.rs:586-625): top-k 8 at temperature 0.8 and full-vocabulary block
sampling at temperature 1.0, each with its LCG seed, and the 8 streams of one 8-sample top-k request.

A third file (c3_600m_bf16_8samples.npz) is the multi-sample workload at its own shape: 512-token
prompt, bf16 KV cache, 8 samples of 256 steps, top-k 8 at temperature 0.8, seeds seed .. seed + 7
(inference.rs:256).  Over 2 040 draws with a bf16 cache some uniform always falls closer to a
threshold of the cumulative weights than the logit tolerance resolves, so equality of whole streams
is not a usable check; the file instead records, for every row and step, what a backend that is fed
the oracle's tokens must reproduce: the merged candidates (ids, values), the gap to the ninth
logit, the drawn token and how far the draw was from the nearest threshold.
Run from the repository root:  python tests/golden/make_fullsize_vectors.py [c2|c3]
"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle_lib as O  # noqa: E402
from rustane_amd import synth  # noqa: E402

CASES = [
    # name, config factory, weight std, weight seed, prompt seed, prompt tokens, greedy steps, bf16 KV cache
    ("c2_600m_bf16_std002", "config_600m", 0.02, 1234, 7, 128, 256, True),
    ("c2_600m_bf16_std005_kvf32", "config_600m", 0.05, 1234, 7, 128, 256, False),
]


SAMPLED = [(0.8, 8, 21), (1.0, 0, 22)]      # temperature, top_k, seed
SAMPLED_STEPS = 24
BATCH = (0.8, 8, 30, 8, 12)                 # temperature, top_k, first seed, samples, steps
C3 = dict(name="c3_600m_bf16_8samples", config="config_600m", weight_std=0.05, weight_seed=1234, prompt_seed=7,
          prompt_tokens=512, temperature=0.8, top_k=8, seed=30, samples=8, steps=256)


def greedy_with_gaps(orc, first, steps):
    """The greedy branch of the cached loop (inference.rs:576-585) step by step, also returning the
    smallest gap between the largest and the second largest logit of any step."""
    tok, out, gap = first, [first], np.inf
    for _ in range(steps - 1):
        lg = orc.decode_logits_from_id(tok)
        tok = int(O.argmax_lower(lg))
        two = np.partition(lg, -2)[-2:]
        gap = min(gap, float(two[1] - two[0]))
        out.append(tok)
    return out, gap


def make_c3():
    """The multi-sample workload with the oracle's tokens, candidates and draw margins per step."""
    t0 = time.time()
    c = C3
    cfg = getattr(synth, c["config"])()
    w = synth.make_weights(cfg, seed=c["weight_seed"], std=c["weight_std"], round_bf16=True)
    ids = synth.make_prompt(c["prompt_seed"], cfg.vocab, c["prompt_tokens"])
    orc = O.Oracle(cfg, w, kv_round_bf16=True)
    lg, _, _ = orc.forward_window(ids)
    lg = lg[0]
    print("c3: prompt forward done in %.1f s" % (time.time() - t0), flush=True)
    top = np.lexsort((np.arange(lg.size), -lg))[:32]
    R, S, K, T = c["samples"], c["steps"], c["top_k"], c["temperature"]
    streams = np.zeros((R, S), np.uint32)
    cand_ids = np.zeros((R, S - 1, K), np.uint32)
    cand_vals = np.zeros((R, S - 1, K), np.float32)
    ninth_gap = np.zeros((R, S - 1), np.float32)
    margin = np.zeros((R, S - 1), np.float32)
    rng_after = np.zeros(R, np.uint64)
    L = O.lib()
    for r in range(R):
        orc.set_len(c["prompt_tokens"])
        rng = O.Rng(c["seed"] + r)
        cur = int(L.orc_sample_next(O.P(O.f32(lg)), cfg.vocab, T, K, rng.ref))       # inference.rs:567-574
        streams[r, 0] = cur
        for i in range(1, S):
            raw = orc.decode_logits_from_id(cur)
            ci, cv = O.topk_candidates(raw, K, 0.0)                                  # inference.rs:586-599
            assert ci.size == K
            cand_ids[r, i - 1], cand_vals[r, i - 1] = ci, cv
            nine = np.partition(raw, -(K + 1))[-(K + 1):]
            nine.sort()
            ninth_gap[r, i - 1] = nine[1] - nine[0]
            wgt = np.exp((cv.astype(np.float64) - float(cv.max())) / T)
            u = O.Rng(rng.s.value).next_f32()
            x = float(u) * wgt.sum()
            margin[r, i - 1] = np.abs(np.cumsum(wgt) - x).min() / wgt.sum()
            cur = int(L.orc_sample_topk_candidates(O.PU(ci), O.P(cv), K, T, rng.ref))
            streams[r, i] = cur
        rng_after[r] = rng.s.value
        print("c3: row %d done at %.1f s" % (r, time.time() - t0), streams[r, :6], flush=True)
    # the hand-written loop above is the reference's cached loop: one row against orc_run_cached_sample
    orc.set_len(c["prompt_tokens"])
    chk, _ = orc.run_cached_sample(ids, lg, 40, T, K, seed=c["seed"] + 2)
    assert [int(t) for t in chk] == [int(t) for t in streams[2, :40]]
    meta = dict(c)
    meta.update({"weights": "bf16-rounded", "kv_cache": "bf16", "prompt_head": [int(x) for x in ids[:8]],
                 "logit_abs_sum": float(np.abs(lg.astype(np.float64)).sum()), "logit_abs_max": float(np.abs(lg).max())})
    np.savez_compressed(os.path.join(HERE, c["name"] + ".npz"), meta=np.array(json.dumps(meta)),
                        top_logit_indices=top.astype(np.uint32), top_logit_values=lg[top].astype(np.float32),
                        streams=streams, cand_ids=cand_ids, cand_vals=cand_vals, ninth_gap=ninth_gap, draw_margin=margin,
                        rng_after=rng_after)
    print("c3 done in %.1f s; smallest draw margin %.2e, smallest ninth gap %.2e" %
          (time.time() - t0, margin.min(), ninth_gap.min()), flush=True)


def main():
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    if which in ("all", "c3"):
        make_c3()
    if which == "c3":
        return
    for name, factory, std, wseed, pseed, n_prompt, steps, kv_bf16 in CASES:
        t0 = time.time()
        cfg = getattr(synth, factory)()
        w = synth.make_weights(cfg, seed=wseed, std=std, round_bf16=True)
        orc = O.Oracle(cfg, w, kv_round_bf16=kv_bf16)
        ids = synth.make_prompt(pseed, cfg.vocab, n_prompt)
        lg, _, _ = orc.forward_window(ids)
        lg = lg[0]
        top = np.lexsort((np.arange(lg.size), -lg))[:32]
        sampled, gap = greedy_with_gaps(orc, int(O.argmax_last(lg)), steps)
        orc.set_len(n_prompt)
        chk, _ = orc.run_cached_sample(ids, lg, 32)         # the step-by-step loop is the reference's cached loop
        assert [int(t) for t in chk] == sampled[:32]
        streams = []
        if not kv_bf16:
            for temperature, top_k, seed in SAMPLED:
                o2 = O.Oracle(cfg, w, kv_round_bf16=kv_bf16)
                o2.forward_window(ids)
                st, _ = o2.run_cached_sample(ids, lg, SAMPLED_STEPS, temperature, top_k, seed=seed)
                streams.append({"temperature": temperature, "top_k": top_k, "seed": seed, "stream": [int(t) for t in st]})
        out = {
            "workload": name, "config": factory, "weight_std": std, "weight_seed": wseed, "prompt_seed": pseed,
            "prompt_tokens": n_prompt, "weights": "bf16-rounded", "kv_cache": "bf16" if kv_bf16 else "f32",
            "prompt_head": [int(x) for x in ids[:8]],
            "top_logit_indices": [int(i) for i in top],
            "top_logit_values": [float(lg[i]) for i in top],
            "logit_abs_sum": float(np.abs(lg.astype(np.float64)).sum()),
            "logit_abs_max": float(np.abs(lg).max()),
            "greedy_stream": [int(t) for t in sampled],
            "greedy_min_top2_gap": gap,
        }
        if streams:
            out["sampled_streams"] = streams
            # the multi-sample workload's shape: 8 samples of one request, seeds seed .. seed + 7 (inference.rs:256)
            temperature, top_k, seed, samples, bsteps = BATCH
            rows = []
            for i in range(samples):
                o2 = O.Oracle(cfg, w, kv_round_bf16=kv_bf16)
                o2.forward_window(ids)
                st, _ = o2.run_cached_sample(ids, lg, bsteps, temperature, top_k, seed=seed + i)
                rows.append([int(t) for t in st])
            out["batch_sampled"] = {"temperature": temperature, "top_k": top_k, "seed": seed, "samples": samples, "streams": rows}
        with open(os.path.join(HERE, name + ".json"), "w") as f:
            json.dump(out, f, indent=1)
        print(name, "done in %.1f s" % (time.time() - t0), out["greedy_stream"][:8], flush=True)


if __name__ == "__main__":
    main()
