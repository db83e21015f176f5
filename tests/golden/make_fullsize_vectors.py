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
and the greedy stream; the fp32-cache case also holds two sampled streams of the reference's cached
loop (crates/engine/src/inference.rs:586-625): top-k 8 at temperature 0.8 and full-vocabulary block
sampling at temperature 1.0, each with its LCG seed, and the 8 streams of one 8-sample top-k request.
Run from the repository root:  python tests/golden/make_fullsize_vectors.py
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
    ("c2_600m_bf16_std002", "config_600m", 0.02, 1234, 7, 128, 24, True),
    ("c2_600m_bf16_std005_kvf32", "config_600m", 0.05, 1234, 7, 128, 24, False),
]


SAMPLED = [(0.8, 8, 21), (1.0, 0, 22)]      # temperature, top_k, seed
BATCH = (0.8, 8, 30, 8, 12)                 # temperature, top_k, first seed, samples, steps


def main():
    for name, factory, std, wseed, pseed, n_prompt, steps, kv_bf16 in CASES:
        t0 = time.time()
        cfg = getattr(synth, factory)()
        w = synth.make_weights(cfg, seed=wseed, std=std, round_bf16=True)
        orc = O.Oracle(cfg, w, kv_round_bf16=kv_bf16)
        ids = synth.make_prompt(pseed, cfg.vocab, n_prompt)
        lg, _, _ = orc.forward_window(ids)
        lg = lg[0]
        top = np.lexsort((np.arange(lg.size), -lg))[:32]
        sampled, _ = orc.run_cached_sample(ids, lg, steps)
        streams = []
        if not kv_bf16:
            for temperature, top_k, seed in SAMPLED:
                o2 = O.Oracle(cfg, w, kv_round_bf16=kv_bf16)
                o2.forward_window(ids)
                st, _ = o2.run_cached_sample(ids, lg, steps, temperature, top_k, seed=seed)
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
