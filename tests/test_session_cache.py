"""The session cache of the reference's server (crates/engine/src/bin/serve.rs:225-471: exact hit,
longest cached prefix + suffix prefill, new session, LRU eviction, window normalisation), with the
HIP backend underneath.  The two unit tests of the reference (serve.rs:1291-1344) are mirrored; the
others check that whatever path the cache takes, the streams are those of a fresh session."""
import numpy as np
import pytest

from rustane_amd import engine as E
from rustane_amd import synth
from rustane_amd.hipdec import Config


def tiny_cfg(seq=64, vocab=1000):
    # inference.rs:929-944 / serve.rs:1296-1306
    return Config.make(dim=256, hidden=640, heads=2, hd=128, seq=seq, nlayers=2, vocab=vocab)


def test_normalize_prompt_ids_keeps_last_seq_window():
    # serve.rs:1320-1344 (no session is created: runs without a GPU)
    cfg = tiny_cfg(seq=64)
    w = synth.make_weights(cfg, seed=3, std=0.02)
    cache = E.SessionCache(cfg, w, max_entries=2)
    np.testing.assert_array_equal(cache.normalize_prompt_ids([1, 2, 3]), [1, 2, 3])
    long_prompt = np.arange(cfg.seq + 5, dtype=np.uint32)
    np.testing.assert_array_equal(cache.normalize_prompt_ids(long_prompt), long_prompt[5:])
    np.testing.assert_array_equal(cache.normalize_prompt_ids(np.arange(cfg.seq, dtype=np.uint32)), np.arange(cfg.seq))
    assert len(cache) == 0 and cache.max_entries() == 2
    assert E.SessionCache(cfg, w, max_entries=0).max_entries() == 1               # serve.rs:267
    assert cache.find_exact([1, 2]) == -1 and cache.find_longest_prefix([1, 2]) == -1


@pytest.mark.gpu
def test_longest_prefix_match_prefers_deepest_entry():
    # serve.rs:1291-1318
    cfg = tiny_cfg()
    w = synth.make_weights(cfg, seed=3, std=0.02)
    cache = E.SessionCache(cfg, w, max_entries=4)
    cache.insert([1, 2])
    cache.insert([1, 2, 3, 4])
    cache.insert([9, 9])
    idx = cache.find_longest_prefix([1, 2, 3, 4, 5])
    assert idx >= 0
    np.testing.assert_array_equal(cache.entry_prompt(idx), [1, 2, 3, 4])
    assert cache.find_longest_prefix([1, 2, 7]) == cache.find_exact([1, 2])
    assert cache.find_longest_prefix([2, 1]) == -1
    assert cache.find_exact([1, 2, 3]) == -1


@pytest.mark.gpu
@pytest.mark.parametrize("T,k", [(0.0, 0), (0.8, 4), (1.0, 0)])
def test_every_cache_path_gives_the_streams_of_a_fresh_session(T, k):
    cfg = tiny_cfg()
    w = synth.make_weights(cfg, seed=31, std=0.08, round_bf16=True)
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=8, temperature=T, top_k=k, samples=2, seed=11)
    cache = E.SessionCache(cfg, w, max_entries=3, weight_dtype=1)

    def fresh(prompt):
        return E.InferenceSession(cfg, w, prompt, weight_dtype=1).generate(req)

    def same(got, want):
        assert len(got.batch.results) == len(want.results) == 2
        for a, b in zip(got.batch.results, want.results):
            np.testing.assert_array_equal(a.sampled, b.sampled)
            np.testing.assert_array_equal(a.generated, b.generated)
            assert a.seed == b.seed

    base, longer, other = [1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 5, 6, 7, 8, 9], [40, 41, 42]
    g = cache.generate(base, req)                                  # miss: new session
    assert (g.cache_prefix_tokens, g.effective_prompt_tokens, g.prompt_truncated, len(cache)) == (0, 6, False, 1)
    same(g, fresh(base))
    g = cache.generate(base, req)                                  # exact hit: nothing to prefill
    assert g.cache_prefix_tokens == 6 and len(cache) == 1
    assert g.batch.request_prefill_elapsed == 0.0
    same(g, fresh(base))
    g = cache.generate(longer, req)                                # extends a cached prompt: only the suffix is prefilled
    assert g.cache_prefix_tokens == 6 and g.effective_prompt_tokens == 9 and len(cache) == 2
    same(g, fresh(longer))
    np.testing.assert_array_equal(cache.entry_prompt(cache.find_exact(longer)), longer)
    one = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=8, temperature=T, top_k=k, samples=1, seed=11)
    g = cache.generate(longer, one, stream=True)                   # now an exact hit, streamed (one sample: inference.rs:330-332)
    assert g.cache_prefix_tokens == 9 and len(g.batch.results) == 1
    want = E.InferenceSession(cfg, w, longer, weight_dtype=1).generate(one)
    np.testing.assert_array_equal(g.batch.results[0].sampled, want.results[0].sampled)
    with pytest.raises(E.SessionError, match="streaming only supports samples=1"):
        cache.generate(longer, req, stream=True)
    g = cache.generate(other, req)
    assert g.cache_prefix_tokens == 0 and len(cache) == 3
    same(g, fresh(other))
    # a fourth prompt evicts the least recently used entry (`base`, last touched before `longer` and `other`)
    g = cache.generate([70, 71], req)
    assert len(cache) == 3 and cache.find_exact(base) == -1
    assert cache.find_exact(longer) >= 0 and cache.find_exact(other) >= 0 and cache.find_exact([70, 71]) >= 0
    same(g, fresh([70, 71]))


@pytest.mark.gpu
def test_long_prompts_are_cut_to_the_window_and_errors_come_back():
    cfg = tiny_cfg(seq=32)
    w = synth.make_weights(cfg, seed=5, std=0.08, round_bf16=True)
    cache = E.SessionCache(cfg, w, max_entries=2, weight_dtype=1)
    req = E.GenerationRequest(E.DecodeBackendRequest.NAIVE, steps=3, temperature=0.0)
    prompt = (np.arange(40) % 50 + 1).astype(np.uint32)
    g = cache.generate(prompt, req)
    assert g.prompt_truncated and g.effective_prompt_tokens == 32
    np.testing.assert_array_equal(cache.entry_prompt(0), prompt[8:])
    want = E.InferenceSession(cfg, w, prompt[8:], weight_dtype=1).generate(req)
    np.testing.assert_array_equal(g.batch.results[0].sampled, want.results[0].sampled)
    with pytest.raises(E.SessionError):
        cache.generate([5, 5000], req)                             # token id beyond the vocabulary (inference.rs:736-749)
    with pytest.raises(E.SessionError):
        cache.generate([], req)                                    # inference.rs:131-133
    assert len(cache) == 1
