"""Where one decode step spends its time: per-phase time stamps of workgroup 0 of the persistent
step kernel, averaged over the middle layers and several steps.

    python3 -m rustane_amd.step_profile [--model 600m|5b] [--weights bf16|fp8|int4] [--prompt N] [--steps K]
    python3 -m rustane_amd.step_profile --rows R [--prompt N]        (multi-sample step, layers as one launch)

Prints the decode time per token of a greedy run, then the cumulative stamps of one layer (in
microseconds from the layer's start) and their differences.  Per layer the stamps are, in order:
qkv phase (start, input staged, first round multiplied, rows finished, end), wo phase (start, q/k/v
arrived, attention done, partials folded, first round multiplied, rows published, end), w13 phase
(five, as qkv), w2 phase (start, gate staged, first round multiplied, rows published, end).
Workgroups that take no attention item skip the two attention stamps.

With --rows R (1 - 8, 600M bf16 model) the profiled launch is the one that runs the layers of a multi-sample
step for R rows stepped together (hipdec_rows.h); its stamps per layer: start, rows of x staged, q/k/v partial
tiles written, q/k/v published, the attention item's q/k/v arrived, attention partial published, folded
attention output staged, output projection multiplied, x2 published, second half's start, rows of x2 staged,
gate / up multiplied, gate published, gate staged, down projection multiplied, x published.
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
    ap.add_argument("--rows", type=int, default=0, help="profile the multi-sample step of this many rows instead")
    args = ap.parse_args()
    if args.rows:
        return rows_profile(args)
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


ROWS_STAMPS = ["start", "x staged", "qkv multiplied", "qkv published", "item's qkv arrived", "partial published",
               "attention output staged", "wo multiplied", "x2 published", "second half", "x2 staged", "w13 multiplied",
               "gate published", "gate staged", "w2 multiplied", "x published", "next layer"]


def rows_profile(args):
    cfg = synth.config_600m()
    w = synth.make_weights(cfg, round_bf16=True)
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    n_prompt = args.prompt if args.prompt != 128 else 512
    dev.prefill(synth.make_prompt(7, cfg.vocab, n_prompt), want_logits=False)
    dev.batch_begin(args.rows)
    if not dev.batch_layers_in_one_launch():
        raise SystemExit("this row count does not run its layers as one launch")
    toks = np.arange(1, args.rows + 1, dtype=np.uint32)
    for _ in range(20):
        toks = dev.decode_token_argmax_from_ids_batch(toks)
    acc = []
    for _ in range(6):
        pr = dev.debug_batch_step_profile(toks).astype(np.int64)
        for l in range(2, cfg.nlayers - 1):
            d = (pr[l][:16] - pr[l][0]) / 100.0          # the wall clock counts at 100 MHz
            acc.append(np.concatenate([d, [(pr[l + 1][0] - pr[l][0]) / 100.0]]))
    mean = np.array(acc).mean(0)
    prev = 0.0
    for name, v in zip(ROWS_STAMPS, mean):
        print("%-26s %7.2f  (+%.2f)" % (name, v, v - prev))
        prev = v
    print("launch %.1f us" % ((pr[cfg.nlayers][0] - pr[0][0]) / 100.0))


if __name__ == "__main__":
    main()
