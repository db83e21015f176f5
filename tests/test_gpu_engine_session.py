"""GPU: the session API (InferenceSession / generate / generate_with_suffix / streaming) over the HIP
backend, against the oracle's restatement of the reference's token loops
(crates/engine/src/inference.rs:542-734) and the reference's own session tests (:976-1033)."""
import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import engine as E
from rustane_amd import synth
from rustane_amd.hipdec import Config

pytestmark = pytest.mark.gpu


def tiny_cfg(vocab=8192, seq=64):
    # inference.rs:929-944
    return Config.make(dim=256, hidden=640, heads=2, hd=128, seq=seq, nlayers=2, vocab=vocab)


def make(cfg, prompt, seed=31, std=0.08, softcap=0.0):
    w = synth.make_weights(cfg, seed=seed, std=std)
    return w, E.InferenceSession(cfg, w, prompt, softcap=softcap)


def oracle_streams(cfg, w, prompt, req, softcap=0.0, suffix=()):
    """What the reference's cached loop yields for every sample of the request."""
    out = []
    full = list(prompt) + list(suffix)
    for i in range(req.samples):
        orc = O.Oracle(cfg, w)
        lg, _, _ = orc.forward_window(np.array(full, np.uint32), softcap=softcap)
        sampled, gen = orc.run_cached_sample(np.array(full, np.uint32), lg[0], req.steps, req.temperature, req.top_k,
                                             seed=req.seed + i, softcap=softcap)
        out.append((sampled, gen))
    return out


@pytest.mark.parametrize("T,k,softcap", [(0.0, 0, 0.0), (0.8, 4, 0.0), (0.8, 8, 3.0), (1.0, 0, 0.0), (1.0, 0, 2.5),
                                         (0.9, 40, 0.0), (0.7, 1, 0.0)])
def test_cached_streams_match_the_oracle_loop(T, k, softcap):
    cfg = tiny_cfg(vocab=1000)
    prompt = [1, 2, 3, 4]
    w, s = make(cfg, prompt, softcap=softcap)
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=12, temperature=T, top_k=k, samples=2, seed=7)
    got = s.generate(req)
    assert got.decode_selection.mode == E.DecodeMode.KV_CACHE_HIP
    want = oracle_streams(cfg, w, prompt, req, softcap)
    assert len(got.results) == 2
    for r, (sampled, gen) in zip(got.results, want):
        np.testing.assert_array_equal(r.sampled, sampled)
        np.testing.assert_array_equal(r.generated, gen)
    assert got.results[0].seed == 7 and got.results[1].seed == 8                 # inference.rs:256
    assert got.total_elapsed == pytest.approx(got.prefill_elapsed + got.total_decode_elapsed)


def test_session_reuses_prompt_across_calls_with_stable_results():
    # inference.rs:976-999
    cfg = tiny_cfg()
    w, s = make(cfg, [1, 2, 3, 4])
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=8, temperature=0.8, top_k=4, samples=2, seed=7)
    first, second = s.generate(req), s.generate(req)
    assert len(first.results) == 2
    for a, b in zip(first.results, second.results):
        np.testing.assert_array_equal(a.generated, b.generated)


def test_session_suffix_matches_fresh_full_prompt_generation():
    # inference.rs:1001-1033
    cfg = tiny_cfg()
    w = synth.make_weights(cfg, seed=31, std=0.08)
    base, suffix = [1, 2, 3], [4, 5]
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=6, temperature=0.8, top_k=4, samples=2, seed=17)
    extended = E.InferenceSession(cfg, w, base).generate_with_suffix(req, suffix)
    fresh = E.InferenceSession(cfg, w, base + suffix).generate(req)
    assert len(extended.results) == len(fresh.results) == 2
    for a, b in zip(extended.results, fresh.results):
        np.testing.assert_array_equal(a.generated, b.generated)
        np.testing.assert_array_equal(a.sampled, b.sampled)
    assert extended.request_prefill_elapsed > 0 and fresh.request_prefill_elapsed == 0


@pytest.mark.parametrize("T,k", [(0.0, 0), (0.8, 4)])
def test_naive_backend_equals_cached_backend(T, k):
    # greedy and top-k<=32 draw once per token on both paths, so the streams coincide
    cfg = tiny_cfg(vocab=1000)
    w, s = make(cfg, [9, 8, 7])
    a = s.generate(E.GenerationRequest(E.DecodeBackendRequest.NAIVE, steps=9, temperature=T, top_k=k, seed=3))
    b = s.generate(E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=9, temperature=T, top_k=k, seed=3))
    c = s.generate(E.GenerationRequest(E.DecodeBackendRequest.NAIVE, steps=9, temperature=T, top_k=k, seed=3))
    assert a.decode_selection.mode == E.DecodeMode.NAIVE_FULL_CONTEXT
    assert b.decode_selection.mode == E.DecodeMode.KV_CACHE_HIP
    np.testing.assert_array_equal(a.results[0].sampled, b.results[0].sampled)
    np.testing.assert_array_equal(a.results[0].sampled, c.results[0].sampled)
    orc = O.Oracle(cfg, w)
    lg, _, _ = orc.forward_window(np.array([9, 8, 7], np.uint32))
    sampled, _ = orc.run_naive_sample(np.array([9, 8, 7], np.uint32), lg[0], 9, T, k, seed=3)
    np.testing.assert_array_equal(a.results[0].sampled, sampled)


def test_window_overflow_falls_back_and_slides():
    cfg = tiny_cfg(vocab=1000, seq=16)
    w, s = make(cfg, [1, 2, 3, 4, 5, 6, 7, 8, 9, 10])
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=12, temperature=0.0)
    got = s.generate(req)
    assert got.decode_selection.mode == E.DecodeMode.NAIVE_FULL_CONTEXT
    assert got.decode_selection.fallback_reason == "requested_length_exceeds_cfg_seq"
    orc = O.Oracle(cfg, w)
    prompt = np.arange(1, 11, dtype=np.uint32)
    lg, _, _ = orc.forward_window(prompt)
    sampled, _ = orc.run_naive_sample(prompt, lg[0], 12, 0.0, 0, seed=1)       # slides once 16 ids are exceeded
    np.testing.assert_array_equal(got.results[0].sampled, sampled)
    one = s.generate(E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=1))
    assert one.decode_selection.fallback_reason == "single_step_prefers_naive"
    assert one.results[0].sampled.tolist() == [int(O.argmax_last(lg[0]))]
    zero = s.generate(E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=0))
    assert zero.decode_selection.mode == E.DecodeMode.PREFILL_ONLY and zero.results[0].sampled.size == 0


def test_streaming_equals_batch_and_callback_error_aborts():
    # inference.rs:321-451, :571-573
    cfg = tiny_cfg(vocab=1000)
    w, s = make(cfg, [4, 5, 6])
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=10, temperature=0.0, seed=5)
    batch = s.generate(req)
    streamed = s.generate_stream_with_suffix(req, [])
    np.testing.assert_array_equal(batch.results[0].sampled, streamed.results[0].sampled)
    assert s.stream_count() == 10
    with pytest.raises(E.SessionError, match="callback asked to stop"):
        s.generate_stream_with_suffix(req, [], abort_after=4)
    assert s.stream_count() == 4
    with pytest.raises(E.SessionError, match="streaming only supports samples=1"):
        s.generate_stream_with_suffix(E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=4, samples=2), [])
    # the session is still usable afterwards
    again = s.generate(req)
    np.testing.assert_array_equal(batch.results[0].sampled, again.results[0].sampled)


def test_session_errors():
    cfg = tiny_cfg(vocab=1000)
    w = synth.make_weights(cfg, seed=31, std=0.08)
    with pytest.raises(E.SessionError, match="prompt must contain at least one token"):
        E.InferenceSession(cfg, w, [])
    with pytest.raises(E.SessionError, match="prompt token id 1000 at position 1 exceeds model vocab 1000"):
        E.InferenceSession(cfg, w, [1, 1000])
    s = E.InferenceSession(cfg, w, [1, 2])
    with pytest.raises(E.SessionError, match="samples must be >= 1"):
        s.generate(E.GenerationRequest(samples=0))
    with pytest.raises(E.SessionError, match="prompt suffix token id 5000"):
        s.generate_with_suffix(E.GenerationRequest(), [5000])


@pytest.mark.parametrize("T,k,softcap", [(0.0, 0, 0.0), (0.8, 8, 0.0), (0.8, 4, 3.0), (1.0, 0, 2.5), (0.9, 40, 0.0)])
def test_samples_stepped_together_equal_sequential_samples(T, k, softcap):
    # The reference draws its samples one after the other (inference.rs:247-262); with bf16 weights
    # this backend advances them together.  Both orders, and the oracle's loop, must give each
    # sample the same stream.
    cfg = tiny_cfg(vocab=1000)
    prompt = [5, 6, 7, 8, 9, 10, 11, 12, 13]
    w = synth.make_weights(cfg, seed=31, std=0.08, round_bf16=True)
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=10, temperature=T, top_k=k, samples=3, seed=21)
    together = E.InferenceSession(cfg, w, prompt, softcap=softcap, weight_dtype=1).generate(req)
    one_by_one = E.InferenceSession(cfg, w, prompt, softcap=softcap, weight_dtype=1, flags=0x100).generate(req)
    want = oracle_streams(cfg, w, prompt, req, softcap)
    assert len(together.results) == len(one_by_one.results) == 3
    for a, b, (sampled, gen) in zip(together.results, one_by_one.results, want):
        np.testing.assert_array_equal(a.sampled, b.sampled)
        np.testing.assert_array_equal(a.sampled, sampled)
        np.testing.assert_array_equal(a.generated, gen)
        assert a.seed == b.seed
    assert together.total_decode_elapsed > 0


def test_f32_weight_samples_step_together_too():
    cfg = tiny_cfg(vocab=1000)
    prompt = [5, 6, 7, 8, 9, 10, 11, 12, 13]
    w = synth.make_weights(cfg, seed=33, std=0.08, round_bf16=False)
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=8, temperature=0.8, top_k=8, samples=3, seed=4)
    together = E.InferenceSession(cfg, w, prompt, weight_dtype=0).generate(req)
    one_by_one = E.InferenceSession(cfg, w, prompt, weight_dtype=0, flags=0x100).generate(req)
    want = oracle_streams(cfg, w, prompt, req, 0.0)
    for a, b, (sampled, gen) in zip(together.results, one_by_one.results, want):
        np.testing.assert_array_equal(a.sampled, b.sampled)
        np.testing.assert_array_equal(a.sampled, sampled)
        np.testing.assert_array_equal(a.generated, gen)


def test_samples_stepped_together_after_a_suffix():
    cfg = tiny_cfg()
    w = synth.make_weights(cfg, seed=31, std=0.08, round_bf16=True)
    base, suffix = [1, 2, 3, 4, 5, 6, 7, 8], [9, 10]
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=6, temperature=0.8, top_k=4, samples=4, seed=17)
    s = E.InferenceSession(cfg, w, base, weight_dtype=1)
    extended = s.generate_with_suffix(req, suffix)
    fresh = E.InferenceSession(cfg, w, base + suffix, weight_dtype=1, flags=0x100).generate(req)
    for a, b in zip(extended.results, fresh.results):
        np.testing.assert_array_equal(a.generated, b.generated)
    # the session's prompt cache survives the batch: a second request gives the same streams
    again = s.generate_with_suffix(req, suffix)
    for a, b in zip(extended.results, again.results):
        np.testing.assert_array_equal(a.sampled, b.sampled)
