"""The line protocol of `generate --jsonl-session` (crates/engine/src/bin/generate.rs:39-144,
:336-491): request parsing with command-line defaults and the reference's rejections on the CPU;
on the GPU the binary is driven through a pipe and its answers are compared with direct session
calls (prefix reuse: the base prompt is prefilled once, appended ids per request)."""
import json
import os
import subprocess

import numpy as np
import pytest

from rustane_amd import engine, synth
from rustane_amd.hipdec import Config

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GENERATE = os.path.join(ROOT, "rustane_amd", "lib", "generate")


def test_request_fields_override_defaults():
    d = engine.GenerationRequest(engine.DecodeBackendRequest.AUTO, steps=20, temperature=0.5, top_k=4, samples=2, seed=9)
    req, sfx = engine.parse_jsonl_request("{}", d)
    assert (req.decode_backend, req.steps, req.temperature, req.top_k, req.samples, req.seed) == \
           (engine.DecodeBackendRequest.AUTO, 20, 0.5, 4, 2, 9) and sfx.size == 0
    line = ' {"append_prompt_ids":[5, 6,7],"decode_backend":"naive","steps":3,"temperature":0.25,' \
           '"top_k":8,"samples":1,"seed":18446744073709551615,"unknown":{"a":[1,"x",null]},"add_special_tokens":true} '
    req, sfx = engine.parse_jsonl_request(line, d)
    assert (req.decode_backend, req.steps, req.temperature, req.top_k, req.samples, req.seed) == \
           (engine.DecodeBackendRequest.NAIVE, 3, 0.25, 8, 1, 2 ** 64 - 1)
    assert sfx.tolist() == [5, 6, 7]
    # Option<T>: null means "not given"; an empty id list is an empty suffix (generate.rs:123-128)
    req, sfx = engine.parse_jsonl_request('{"steps":null,"append_prompt_ids":[],"seed":null}', d)
    assert (req.steps, req.seed, sfx.size) == (20, 9, 0)


def test_request_rejections():
    def msg(line):
        with pytest.raises(engine.JsonlRequestError) as e:
            engine.parse_jsonl_request(line)
        return str(e.value)

    assert msg("not json").startswith("invalid json request: ")
    assert msg('{"steps":-1}').startswith("invalid json request: ")
    assert msg('{"steps":1.5}').startswith("invalid json request: ")
    assert msg('{"append_prompt_ids":[1,4294967296]}').startswith("invalid json request: ")
    assert msg('{"steps":3} trailing').startswith("invalid json request: ")
    assert msg('{"decode_backend":"cuda"}') == "decode_backend must be one of: auto, naive, hip; got cuda"
    assert msg('{"decode_backend":"metal"}').startswith("decode_backend metal is the Apple-GPU backend")
    assert msg('{"samples":0}') == "samples must be >= 1"
    assert msg('{"append_prompt_ids":[1],"append_prompt":"x"}') == "pass either append_prompt_ids or append_prompt, not both"
    assert msg('{"append_prompt":"hello"}') == "append_prompt requires the session to be started with --tokenizer"


@pytest.mark.gpu
def test_binary_session_answers_equal_direct_session_calls(tmp_path):
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w = synth.make_weights(cfg, seed=8, std=0.08, round_bf16=True)
    path = tmp_path / "ckpt_000003.bin"
    engine.write_checkpoint(path, cfg, w, step=3)
    base = [1, 2, 3, 4, 5, 6, 7, 8, 9]
    lines = ['{"steps":6}',
             '{"append_prompt_ids":[11,12,13],"steps":5,"temperature":0.8,"top_k":4,"samples":2,"seed":5}',
             '',
             '{"steps":4,"decode_backend":"naive"}',
             '{"samples":0}',
             '{"append_prompt_ids":[400]}',
             '{"steps":6}']
    proc = subprocess.run([GENERATE, "--checkpoint", str(path), "--prompt-ids", ",".join(map(str, base)), "--jsonl-session",
                           "--decode-backend", "hip", "--weight-dtype", "bf16", "--kv-dtype", "f32"],
                          input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    assert proc.stderr.startswith("jsonl_session_ready checkpoint_step=3 prompt_len=9 decode_backend_default=hip")
    out = [json.loads(l) for l in proc.stdout.splitlines()]
    assert len(out) == 6                                   # the blank line is skipped (generate.rs:437-439)
    assert out[3] == {"error": "samples must be >= 1"}
    assert "error" in out[4] and "400" in out[4]["error"]   # token id outside the vocabulary (inference.rs:736-749)

    sess = engine.InferenceSession(cfg, w, base, weight_dtype=1, kv_dtype=0)
    hip, naive = engine.DecodeBackendRequest.HIP, engine.DecodeBackendRequest.NAIVE
    a = sess.generate(engine.GenerationRequest(hip, steps=6))
    b = sess.generate_with_suffix(engine.GenerationRequest(hip, steps=5, temperature=0.8, top_k=4, samples=2, seed=5), [11, 12, 13])
    c = sess.generate(engine.GenerationRequest(naive, steps=4))
    for got, want, mode, prompt in ((out[0], a, "kv_cache_hip", base), (out[1], b, "kv_cache_hip", base + [11, 12, 13]),
                                    (out[2], c, "naive_full_context", base), (out[5], a, "kv_cache_hip", base)):
        assert got["decode_mode"] == mode and got["base_prompt_ids"] == base and got["prompt_ids"] == prompt
        assert got["base_prompt_text"] is None and got["results"][0]["generated_text"] is None
        assert len(got["results"]) == len(want.results)
        for gr, wr in zip(got["results"], want.results):
            assert gr["seed"] == wr.seed
            assert gr["generated_ids"] == list(map(int, wr.sampled))
            assert gr["full_sequence"] == list(map(int, wr.generated))
    assert out[1]["decode_backend_request"] == "hip" and out[2]["decode_backend_request"] == "naive"
    assert list(out[0]) == ["decode_backend_request", "decode_mode", "fallback_reason", "auto_reason", "base_prompt_ids",
                            "prompt_ids", "base_prompt_text", "prompt_text", "base_prefill_ms", "base_prefill_tok_per_s",
                            "request_prefill_ms", "total_prefill_ms", "request_decode_ms_total", "request_decode_ms_avg",
                            "request_avg_decode_tok_per_s", "end_to_end_ms_including_prefill",
                            "end_to_end_tok_per_s_including_prefill", "results"]
    assert list(out[0]["results"][0]) == ["seed", "generated_ids", "full_sequence", "generated_text", "full_text",
                                          "decode_time_ms", "decode_tok_per_s"]
    assert out[1]["request_prefill_ms"] > 0 and out[0]["request_prefill_ms"] == 0


def _report(stdout):
    """The one-shot report as a list of lines and a dict of its space-separated key=value fields."""
    lines = stdout.splitlines()
    fields = {}
    for ln in lines:
        for part in ln.split(" "):
            if "=" in part:
                k, v = part.split("=", 1)
                fields[k] = v
    return lines, fields


@pytest.mark.gpu
def test_one_shot_report_lines_follow_the_reference(tmp_path):
    """`generate` without --jsonl-session prints the reference's report (generate.rs:524-566 before the run,
    :609-728 after it): same keys, same order, ids equal to a direct session's."""
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w = synth.make_weights(cfg, seed=8, std=0.08, round_bf16=True)
    path = tmp_path / "ckpt_000007.bin"
    engine.write_checkpoint(path, cfg, w, step=7)
    base = [1, 2, 3, 4, 5, 6, 7, 8, 9]
    ids = ",".join(map(str, base))
    common = [GENERATE, "--checkpoint", str(path), "--prompt-ids", ids, "--weight-dtype", "bf16", "--kv-dtype", "f32"]
    sess = engine.InferenceSession(cfg, w, base, weight_dtype=1, kv_dtype=0)
    hip = engine.DecodeBackendRequest.HIP

    # one greedy sample
    proc = subprocess.run(common + ["--steps", "6", "--decode-backend", "hip"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    lines, f = _report(proc.stdout)
    want = sess.generate(engine.GenerationRequest(hip, steps=6)).results[0]
    assert lines[0] == "loaded checkpoint: step=7 model=2L 256D 640H 320V seq=96"
    assert lines[1] == ("prompt_len=9 effective_context_len=9 steps=6 temperature=0 top_k=0 decode_backend_request=hip "
                        "decode_mode=kv_cache_hip greedy_sampling=true")
    assert lines[2] == "samples=1 prefix_reuse=disabled"
    assert lines[3] == "prompt_ids=" + ids
    assert lines[4] == "generated_ids=" + ",".join(str(int(t)) for t in want.sampled)
    assert lines[5] == "full_sequence=" + ",".join(str(int(t)) for t in want.generated)
    assert [ln.split("=")[0] for ln in lines[6:]] == ["prefill_time", "decode_steps", "total_generation_time"]
    assert f["decode_steps"] == "5" and f["prefill_time"].endswith("ms") and f["decode_time"].endswith("ms")
    assert float(f["prefill_tok/s"]) > 0 and float(f["decode_tok/s"]) > 0 and float(f["overall_tok/s"]) > 0
    assert len(lines) == 9

    # two sampled continuations, candidates from the device: per-sample lines and the averages
    proc = subprocess.run(common + ["--steps", "5", "--temperature", "0.8", "--top-k", "4", "--samples", "2", "--seed", "5",
                                    "--decode-backend", "hip"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    lines, f = _report(proc.stdout)
    want = sess.generate(engine.GenerationRequest(hip, steps=5, temperature=0.8, top_k=4, samples=2, seed=5)).results
    assert lines[1] == ("prompt_len=9 effective_context_len=9 steps=5 temperature=0.8 top_k=4 decode_backend_request=hip "
                        "decode_mode=kv_cache_hip greedy_sampling=false")
    assert lines[2] == "samples=2 prefix_reuse=enabled"
    assert lines[3] == "cached_sampling_path=gpu_topk_candidates top_k=4 gpu_topk_capacity=32"
    assert lines[4] == "prompt_ids=" + ids
    at = 5
    for i, r in enumerate(want):
        assert lines[at] == "sample%d_seed=%d" % (i, r.seed)
        assert lines[at + 1] == "sample%d_generated_ids=%s" % (i, ",".join(str(int(t)) for t in r.sampled))
        assert lines[at + 2] == "sample%d_full_sequence=%s" % (i, ",".join(str(int(t)) for t in r.generated))
        assert lines[at + 3].startswith("sample%d_decode_steps=4 sample%d_decode_time=" % (i, i))
        assert " sample%d_decode_tok/s=" % i in lines[at + 3]
        at += 4
    assert [ln.split("=")[0] for ln in lines[at:]] == ["prefill_time", "samples_decode_time_total", "total_generation_time"]
    assert "samples_decode_time_avg" in f and "avg_decode_tok/s" in f
    assert len(lines) == at + 3

    # the planner's notes: auto on a small model, a window that overflows, block statistics, a wide top-k
    proc = subprocess.run(common + ["--steps", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    lines, f = _report(proc.stdout)
    assert f["decode_backend_request"] == "auto" and f["decode_mode"] == "naive_full_context"
    assert lines[2] == "decode_backend_auto_reason=model_param_count_lt_threshold model_params=%d auto_metal_threshold=20000000" % (
        cfg.param_count())
    proc = subprocess.run(common[:4] + [",".join(str(1 + i % 300) for i in range(100)), "--weight-dtype", "bf16", "--steps", "3",
                                        "--decode-backend", "hip"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    lines, f = _report(proc.stdout)
    assert f["prompt_len"] == "100" and f["effective_context_len"] == "96"
    assert lines[2] == "prompt_truncated=true kept_last_tokens=96"
    assert lines[3] == "decode_backend_fallback=true reason=requested_length_exceeds_cfg_seq"
    for extra, note in ((["--temperature", "1.5"], "cached_sampling_path=gpu_block_stats_exact"),
                        (["--temperature", "0.7", "--top-k", "40"],
                         "cached_sampling_path=full_logits_cpu_sample reason=top_k_exceeds_gpu_capacity requested_top_k=40 "
                         "gpu_topk_capacity=32")):
        proc = subprocess.run(common + ["--steps", "3", "--decode-backend", "hip"] + extra, capture_output=True, text=True,
                              timeout=120)
        assert proc.returncode == 0, proc.stderr
        assert note in proc.stdout.splitlines()
