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
