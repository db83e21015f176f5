"""Where one decode step spends its time: per-phase time stamps of workgroup 0 of the persistent
step kernel, averaged over the middle layers and several steps.

    python3 -m rustane_amd.step_profile [--model 600m|5b] [--weights bf16|fp8|int4] [--prompt N] [--steps K]

Prints the decode time per token of a greedy run, then the cumulative stamps of one layer (in
microseconds from the layer's start) and their differences.  Per layer the stamps are, in order:
qkv phase (start, input staged, first round multiplied, rows finished, end), wo phase (start, q/k/v
arrived, attention done, partials folded, first round multiplied, rows published, end), w13 phase
(five, as qkv), w2 phase (start, gate staged, first round multiplied, rows published, end).
Workgroups that take no attention item skip the two attention stamps.
"""
import argparse

import numpy as np

from . import synth
from .hipdec import HipDecodeModel, KvDtype, WeightDtype


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", default="600m", choices=["600m", "5b"])
    ap.add_argument("--weights", default="bf16", choices=["bf16", "fp8", "int4"])
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--steps", type=int, default=255)
    args = ap.parse_args()
    cfg = synth.config_600m() if args.model == "600m" else synth.config_5b()
    wd = {"bf16": WeightDtype.BF16, "fp8": WeightDtype.FP8_E4M3, "int4": WeightDtype.INT4_G128}[args.weights]
    w = synth.make_weights(cfg, round_bf16=True)
    dev = HipDecodeModel(cfg, w, weight_dtype=wd, kv_dtype=KvDtype.BF16)
    prompt = synth.make_prompt(7, cfg.vocab, args.prompt)
    first = int(np.argmax(dev.prefill(prompt)))
    for _ in range(3):
        dev.set_len(args.prompt)
        dev.decode_greedy_run(first, args.steps)
        print("ms per token %.4f" % (dev.last_device_ms() / args.steps), flush=True)
    at = args.prompt + args.steps // 2          # the profiled step attends over the run's mean length
    acc = None
    for _ in range(4):
        dev.set_len(at)
        pr = dev.debug_step_profile(first).astype(np.int64)
        rows = []
        for l in range(2, cfg.nlayers - 1):
            n = int((pr[l] != 0).sum())
            d = (pr[l][:n] - pr[l][0]) / 100.0  # the wall clock counts at 100 MHz
            rows.append(np.concatenate([d, [(pr[l + 1][0] - pr[l][0]) / 100.0]]))
        m = min(len(r) for r in rows)
        a = np.array([r[:m - 1].tolist() + [r[-1]] for r in rows])
        acc = a if acc is None else np.concatenate([acc, a])
    mean = acc.mean(0)
    print("stamps per layer", len(mean) - 1)
    print("cumulative us:", " ".join("%.2f" % v for v in mean))
    print("deltas     us:", " ".join("%.2f" % v for v in np.diff(mean)))
    print("layer period %.2f us" % mean[-1])


if __name__ == "__main__":
    main()
