"""Host-side logic of the engine (backend selection, samplers, RNG, token validation, candidate merge)
checked on the CPU against the reference's own unit tests and against the oracle's restatement."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import engine as E
from rustane_amd.hipdec import Config

L = E.lib()
fp, u32p = E.fp, E.u32p


def tiny_cfg():
    # crates/engine/src/inference.rs:929-944
    return Config.make(dim=256, hidden=640, heads=2, hd=128, seq=64, nlayers=2, vocab=8192)


def gpt_1024():
    # crates/engine/src/model.rs:105-122
    return Config.make(dim=1024, hidden=2816, heads=8, hd=128, seq=512, nlayers=8, vocab=8192)


def test_param_count_matches_formula_and_threshold():
    c = gpt_1024()
    want = 8 * (4 * 1024 * 1024 + 3 * 1024 * 2816) + 8192 * 1024 + 1024 * 17
    assert E.param_count(c) == want == c.param_count()
    assert E.param_count(tiny_cfg()) < E.AUTO_KV_PARAM_THRESHOLD <= want


def test_auto_prefers_naive_on_tiny_model():
    # inference.rs:946-951
    s = E.select_decode_mode(tiny_cfg(), E.DecodeBackendRequest.AUTO, 4, 8)
    assert s.mode == E.DecodeMode.NAIVE_FULL_CONTEXT
    assert s.auto_reason == "model_param_count_lt_threshold"


def test_auto_prefers_kv_cache_on_gpt_1024():
    # inference.rs:953-959
    s = E.select_decode_mode(gpt_1024(), E.DecodeBackendRequest.AUTO, 4, 32)
    assert s.mode == E.DecodeMode.KV_CACHE_HIP
    assert s.auto_reason == "model_param_count_ge_threshold"


def test_forced_gpu_backend_falls_back_when_window_exceeds_seq():
    # inference.rs:961-974
    s = E.select_decode_mode(gpt_1024(), E.DecodeBackendRequest.HIP, 500, 20)
    assert s.mode == E.DecodeMode.NAIVE_FULL_CONTEXT
    assert s.fallback_reason == "requested_length_exceeds_cfg_seq"


def test_select_decode_mode_remaining_branches():
    # inference.rs:464-527, branch by branch
    g = gpt_1024()
    assert E.select_decode_mode(g, E.DecodeBackendRequest.HIP, 4, 0).mode == E.DecodeMode.PREFILL_ONLY
    s = E.select_decode_mode(g, E.DecodeBackendRequest.HIP, 4, 1)
    assert (s.mode, s.fallback_reason) == (E.DecodeMode.NAIVE_FULL_CONTEXT, "single_step_prefers_naive")
    s = E.select_decode_mode(g, E.DecodeBackendRequest.HIP, 4, 508)
    assert (s.mode, s.fallback_reason) == (E.DecodeMode.KV_CACHE_HIP, None)        # 4 + 508 == seq is allowed
    s = E.select_decode_mode(g, E.DecodeBackendRequest.NAIVE, 4, 32)
    assert (s.mode, s.fallback_reason, s.auto_reason) == (E.DecodeMode.NAIVE_FULL_CONTEXT, None, None)
    s = E.select_decode_mode(g, E.DecodeBackendRequest.AUTO, 4, 1)
    assert (s.mode, s.fallback_reason, s.auto_reason) == (E.DecodeMode.NAIVE_FULL_CONTEXT, None,
                                                          "single_step_prefers_naive")
    s = E.select_decode_mode(g, E.DecodeBackendRequest.AUTO, 500, 20)
    assert (s.mode, s.fallback_reason, s.auto_reason) == (E.DecodeMode.NAIVE_FULL_CONTEXT,
                                                          "requested_length_exceeds_cfg_seq",
                                                          "window_not_metal_eligible")


def test_parse_decode_backend():
    # inference.rs:19-34, with `hip` beside the reference's names
    assert E.parse_decode_backend("auto") == E.DecodeBackendRequest.AUTO
    assert E.parse_decode_backend("naive") == E.DecodeBackendRequest.NAIVE
    assert E.parse_decode_backend("hip") == E.DecodeBackendRequest.HIP
    assert E.parse_decode_backend("metal") is None          # the Apple-GPU backend is not an alias of hip
    assert E.parse_decode_backend("cuda") is None


def test_rng_matches_oracle_and_integers():
    s = C.c_uint64(17)
    r = O.Rng(17)
    ref = 17
    for _ in range(6):
        ref = (ref * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        assert L.rs_next_u64(C.byref(s)) == ref == r.next_u64()
    assert L.rs_next_f32(C.byref(s)) == r.next_f32()


def _logits(seed, n, scale=2.0):
    return (scale * np.random.default_rng(seed).standard_normal(n)).astype(np.float32)


@pytest.mark.parametrize("T,k", [(0.0, 0), (0.9, 1), (0.8, 4), (0.8, 40), (1.0, 0), (0.7, 5000), (1.3, 3)])
def test_sample_next_equals_oracle(T, k):
    OL = O.lib()
    for seed in range(40):
        lg = _logits(seed, 777)
        a, b = C.c_uint64(seed * 13 + 1), C.c_uint64(seed * 13 + 1)
        got = L.rs_sample_next(lg.ctypes.data_as(fp), lg.size, T, k, C.byref(a))
        want = OL.orc_sample_next(O.P(lg), lg.size, T, k, C.byref(b))
        assert got == want and a.value == b.value


def test_candidate_and_block_samplers_equal_oracle():
    OL = O.lib()
    for seed in range(60):
        raw = _logits(seed, 1000, 3.0)
        idxs, vals = O.topk_candidates(raw, 8, softcap=0.0)
        a, b = C.c_uint64(seed + 5), C.c_uint64(seed + 5)
        got = L.rs_sample_topk_candidates(idxs.ctypes.data_as(u32p), vals.ctypes.data_as(fp), idxs.size, 0.8, C.byref(a))
        want = OL.orc_sample_topk_candidates(O.PU(idxs), O.P(vals), idxs.size, 0.8, C.byref(b))
        assert got == want and a.value == b.value
        mx, sm = O.block_stats(raw, 1.0 / 0.9, 0.0)
        blk = L.rs_sample_block_from_stats(mx.ctypes.data_as(fp), sm.ctypes.data_as(fp), mx.size, C.byref(a))
        assert blk == OL.orc_sample_block_from_stats(O.P(mx), O.P(sm), mx.size, C.byref(b))
        bl = O.materialize_block(raw, blk, 0.0)
        got = L.rs_sample_block_logits(blk * 256, bl.ctypes.data_as(fp), bl.size, 0.9, C.byref(a))
        want = OL.orc_sample_block_logits(blk * 256, O.P(bl), bl.size, 0.9, C.byref(b))
        assert got == want and a.value == b.value
        assert L.rs_sample_softmax_index(bl.ctypes.data_as(fp), bl.size, 0.9, C.byref(a)) == \
            OL.orc_sample_softmax_index(O.P(bl), bl.size, 0.9, C.byref(b))


def test_sampler_degenerate_cases():
    s = C.c_uint64(1)
    assert L.rs_sample_topk_candidates(None, None, 0, 0.8, C.byref(s)) == 0          # inference.rs:824-826
    mx = np.array([-np.inf, -np.inf], np.float32); sm = np.zeros(2, np.float32)
    assert L.rs_sample_block_from_stats(mx.ctypes.data_as(fp), sm.ctypes.data_as(fp), 2, C.byref(s)) == 0
    x = np.array([0.0, 5.0, 5.0, -1.0], np.float32)
    assert L.rs_sample_next(x.ctypes.data_as(fp), 4, 0.0, 0, C.byref(s)) == 2        # max_by keeps the last maximum
    assert s.value == 1                                                              # greedy draws nothing


@pytest.mark.parametrize("k", [1, 4, 32])
def test_merge_topk_candidates_equals_oracle(k):
    rng = np.random.default_rng(k)
    x = rng.standard_normal(900).astype(np.float32)
    x[rng.integers(0, 900, 30)] = 0.75
    x[3] = np.inf; x[700] = -np.inf
    vals, idxs = O.block_topk(x, k)
    ov = np.empty(k, np.float32); oi = np.empty(k, np.uint32)
    n = L.rs_merge_topk_candidates(vals.ctypes.data_as(fp), idxs.ctypes.data_as(u32p), vals.size, k,
                                   ov.ctypes.data_as(fp), oi.ctypes.data_as(u32p))
    wv, wi = O.merge_topk(vals, idxs, k)
    assert n == wi.size
    np.testing.assert_array_equal(oi[:n], wi)
    np.testing.assert_array_equal(ov[:n], wv)


def test_validate_token_ids_message_and_window():
    ids = np.array([1, 2, 9000, 4], np.uint32)
    err = C.create_string_buffer(256)
    assert L.rs_validate_token_ids(ids.ctypes.data_as(u32p), 4, 8192, b"prompt", err, 256) == 1
    assert err.value.decode() == "prompt token id 9000 at position 2 exceeds model vocab 8192"   # inference.rs:743-746
    assert L.rs_validate_token_ids(ids.ctypes.data_as(u32p), 2, 8192, b"prompt", err, 256) == 0
    gen = np.arange(1, 11, dtype=np.uint32)
    out = np.full(4, 9, np.uint32)
    assert L.rs_fill_input_window(gen.ctypes.data_as(u32p), 10, 4, out.ctypes.data_as(u32p)) == 4
    assert out.tolist() == [7, 8, 9, 10]
    out = np.full(16, 9, np.uint32)
    assert L.rs_fill_input_window(gen.ctypes.data_as(u32p), 10, 16, out.ctypes.data_as(u32p)) == 10
    assert out.tolist() == list(range(1, 11)) + [0] * 6


def test_generate_cli_refuses_text_flags_with_a_clear_message():
    # generate.rs:173-188 takes text through a tokenizer; this build works on token ids only
    import os
    import subprocess
    from rustane_amd import build as B
    if not os.path.exists(B.GENERATE_BIN):
        pytest.skip("generate binary not built")
    for flag in ("--prompt", "--tokenizer"):
        res = subprocess.run([B.GENERATE_BIN, "--model", "tiny", flag, "x"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                             text=True)
        assert res.returncode != 0
        assert "needs a tokenizer" in res.stdout and "--prompt-ids" in res.stdout
    res = subprocess.run([B.GENERATE_BIN, "--frobnicate"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode != 0 and "unknown argument --frobnicate" in res.stdout
