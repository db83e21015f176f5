"""GPU checks at the benchmark models' full sizes, through the C ABI.  Where the CPU oracle is too
slow to replay a whole workload these use properties that do not depend on size: the multi-row
step must agree with single-row steps, the chunked matrix-core prefill with the token-step prefill,
a device-chained greedy run with the same steps taken one call at a time; the 5B-class model is
also checked against the oracle directly on a short prompt."""
import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import synth
from rustane_amd.hipdec import Config, HipDecodeModel, KvDtype, WeightDtype

pytestmark = pytest.mark.gpu
FLAG_PREFILL_STEPS = 4


def rel_err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / max(np.abs(b).max(), 1e-30))


@pytest.fixture(scope="module")
def w600():
    cfg = synth.config_600m()
    return cfg, synth.make_weights(cfg, seed=1234, std=0.05, round_bf16=True)


@pytest.fixture(scope="module")
def w5b():
    cfg = synth.config_5b()
    return cfg, synth.make_weights(cfg, seed=1234, std=0.03, round_bf16=True)


def test_600m_multi_row_step_equals_single_row_steps(w600):
    cfg, w = w600
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    ids = synth.make_prompt(7, cfg.vocab, 512)
    lg = dev.prefill(ids)
    order = np.argsort(-lg, kind="stable")
    rows = 8
    starts = [int(order[r]) for r in range(rows)]
    # sequential: each row alone, three steps, from the shared prompt
    want = []
    for r in range(rows):
        dev.set_len(512)
        tok, seq = starts[r], []
        for _ in range(3):
            l1 = dev.decode_logits_from_id(tok)
            seq.append(l1)
            tok = int(np.argmax(l1))
        want.append(seq)
    dev.set_len(512)
    dev.batch_begin(rows)
    toks = np.array(starts, np.uint32)
    for step in range(3):
        got = dev.decode_logits_from_ids_batch(toks)
        for r in range(rows):
            assert rel_err(got[r], want[r][step]) < 2e-3, (step, r)
        toks = np.array([int(np.argmax(want[r][step])) for r in range(rows)], np.uint32)
    dev.batch_end()
    assert dev.len() == 512


def test_600m_chained_greedy_run_equals_single_calls(w600):
    cfg, w = w600
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    ids = synth.make_prompt(7, cfg.vocab, 128)
    first = int(np.argmax(dev.prefill(ids)))
    run = dev.decode_greedy_run(first, 40)
    dev.set_len(128)
    tok, single = first, []
    for _ in range(40):
        tok = dev.decode_token_argmax_from_id(tok)
        single.append(tok)
    np.testing.assert_array_equal(run, single)
    assert dev.len() == 168


def test_600m_sampled_runs_on_the_device_equal_the_host_loop(w600):
    """The two sampled workloads at the benchmark model's size (128 vocab blocks): tokens drawn on the
    device (hipdec_decode_*_sampled_run*) against the reference's loop -- candidates / statistics
    read back each step, the oracle's merge and draws on the host (inference.rs:586-625)."""
    cfg, w = w600
    a = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    b = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    ids = synth.make_prompt(7, cfg.vocab, 256)
    lg = a.prefill(ids)
    np.testing.assert_array_equal(lg, b.prefill(ids))
    first = int(np.argmax(lg))
    steps = 24
    # top-k 8 at T 0.8 (one draw per token)
    got, state = a.decode_topk_sampled_run(first, 8, 0.8, 1234, steps)
    rng, tok, want = O.Rng(1234), first, []
    for _ in range(steps):
        vals, idxs = b.decode_token_topk_from_id(tok, 8)
        mv, mi = O.merge_topk(vals, idxs, 8)
        tok = int(O.lib().orc_sample_topk_candidates(O.PU(mi), O.P(mv), mi.size, 0.8, rng.ref))
        want.append(tok)
    np.testing.assert_array_equal(got, np.array(want, np.uint32))
    assert state == rng.s.value
    # full vocabulary at T 1.0 (block draw, then token draw), continuing both models
    got, state = a.decode_fullvocab_sampled_run(int(got[-1]), 1.0, 99, steps)
    rng, want = O.Rng(99), []
    for _ in range(steps):
        mx, sm = b.decode_token_block_stats_from_id(tok, 1.0, 0.0)
        blk = int(O.lib().orc_sample_block_from_stats(O.P(mx), O.P(sm), mx.size, rng.ref))
        bl = b.materialize_current_logits_block(blk, 0.0)
        tok = int(O.lib().orc_sample_block_logits(blk * 256, O.P(bl), bl.size, 1.0, rng.ref))
        want.append(tok)
    np.testing.assert_array_equal(got, np.array(want, np.uint32))
    assert state == rng.s.value
    # 8 rows stepped together, top-k 8: every row against its own host loop over the batched candidates
    rows = 8
    a.batch_begin(rows)
    b.batch_begin(rows)
    starts = np.argsort(-lg, kind="stable")[:rows].astype(np.uint32)
    seeds = np.arange(rows, dtype=np.uint64) + np.uint64(5)
    got, states = a.decode_topk_sampled_run_batch(starts, 8, 0.8, seeds, steps)
    rngs, cur = [O.Rng(int(x)) for x in seeds], starts.copy()
    for i in range(steps):
        vals, idxs = b.decode_token_topk_from_ids_batch(cur, 8)
        nxt = np.empty(rows, np.uint32)
        for r in range(rows):
            mv, mi = O.merge_topk(vals[r], idxs[r], 8)
            nxt[r] = O.lib().orc_sample_topk_candidates(O.PU(mi), O.P(mv), mi.size, 0.8, rngs[r].ref)
        np.testing.assert_array_equal(got[i], nxt, err_msg="step %d" % i)
        cur = nxt
    np.testing.assert_array_equal(states, np.array([x.s.value for x in rngs], np.uint64))
    a.batch_end()
    b.batch_end()


@pytest.mark.parametrize("kvdt,tol", [(KvDtype.F32, 2e-4), (KvDtype.BF16, 2e-2)])
def test_5b_bf16_short_prompt_against_the_oracle(w5b, kvdt, tol):
    # fp32 cache: the fp32-path bound (1e-4 at the reference's tiny test shapes, crates/engine/tests/
    # auto_kv_decode.rs:67-215; 2e-4 here for 32 layers of dim 4096).  bf16 cache: the bf16 bound, 2e-2 --
    # 1-ulp differences flip the bf16 rounding of cached values, measured 8e-3 on this model.
    cfg, w = w5b
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=kvdt)
    orc = O.Oracle(cfg, w, kv_round_bf16=(kvdt == KvDtype.BF16))
    ids = synth.make_prompt(7, cfg.vocab, 16)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert rel_err(lg_d, lg_o[0]) < tol
    tok = int(O.argmax_lower(lg_o[0]))
    assert int(np.argmax(lg_d)) == tok
    for _ in range(3):
        a = orc.decode_logits_from_id(tok)
        b = dev.decode_logits_from_id(tok)
        assert rel_err(b, a) < tol
        assert int(np.argmax(b)) == int(O.argmax_lower(a))
        tok = int(O.argmax_lower(a))


@pytest.mark.parametrize("kvdt,tol", [(KvDtype.F32, 2e-4), (KvDtype.BF16, 2e-2)])
def test_5b_shape_long_prompt_many_attention_splits_against_the_oracle(w5b, kvdt, tol):
    """The 5B layer shape (dim 4096, 32 heads of 128, hidden 11008) on the first four layers of the 5B weights, so
    that the CPU oracle can afford a prompt long enough for the token step to deal its attention over several
    workgroups per head (a split covers 64 cache rows with an fp32 cache, 128 with a bf16 one): the chunked
    matrix-core prefill of 260 rows, then token steps whose partial records are folded across 3 to 5 splits at
    dim 4096 / 32 heads, each against the oracle."""
    cfg5, w5 = w5b
    cfg = Config.make(dim=cfg5.dim, hidden=cfg5.hidden, heads=cfg5.heads, hd=cfg5.hd, seq=512, nlayers=4, vocab=cfg5.vocab)
    w = {"embed": w5["embed"], "gamma_final": w5["gamma_final"], "layers": w5["layers"][:4]}
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=kvdt)
    orc = O.Oracle(cfg, w, kv_round_bf16=(kvdt == KvDtype.BF16))
    ids = synth.make_prompt(11, cfg.vocab, 260)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert rel_err(lg_d, lg_o[0]) < tol
    tok = int(O.argmax_lower(lg_o[0]))
    assert int(np.argmax(lg_d)) == tok
    for _ in range(4):
        a = orc.decode_logits_from_id(tok)
        b = dev.decode_logits_from_id(tok)
        assert rel_err(b, a) < tol
        assert int(np.argmax(b)) == int(O.argmax_lower(a))
        tok = int(O.argmax_lower(a))
    assert dev.len() == 264


@pytest.mark.parametrize("wdt", [WeightDtype.FP8_E4M3, WeightDtype.INT4_G128])
def test_5b_quantised_prefill_paths_and_chained_run_agree(w5b, wdt):
    cfg, w = w5b
    ids = synth.make_prompt(7, cfg.vocab, 96)
    a = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=KvDtype.F32)
    la = a.prefill(ids)
    first = int(np.argmax(la))
    run = a.decode_greedy_run(first, 12)
    if wdt == WeightDtype.FP8_E4M3:
        # chunked matrix-core prefill against one token step per prompt row (4-bit weights always use the latter)
        b = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=KvDtype.F32, flags=FLAG_PREFILL_STEPS)
        lb = b.prefill(ids)
        assert rel_err(la, lb) < 2e-4      # fp32 cache: only the accumulation order differs
        assert int(np.argmax(lb)) == first
        del b
    a.set_len(96)
    tok, single = first, []
    for _ in range(12):
        tok = a.decode_token_argmax_from_id(tok)
        single.append(tok)
    np.testing.assert_array_equal(run, single)


def test_5b_bf16_workload_prefill_paths_and_fullvocab_sampled_run(w5b):
    """The 5B bf16 workload at its own shape: 1024-token prompt, bf16 cache, then full-vocabulary
    sampling at temperature 1.0 through the block-statistics path.  (i) The chunked matrix-core
    prefill against one token step per prompt row (the persistent kernel, whose fold covers
    32 heads x up to 8 splits on the way).  (ii) 24 steps of
    hipdec_decode_fullvocab_sampled_run against the reference's loop built from the per-step calls
    and the oracle's two draws (inference.rs:600-625), tokens and RNG state."""
    cfg, w = w5b
    ids = synth.make_prompt(7, cfg.vocab, 1024)
    a = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    b = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    c = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16, flags=FLAG_PREFILL_STEPS)
    la = a.prefill(ids)
    np.testing.assert_array_equal(la, b.prefill(ids))
    lc = c.prefill(ids)
    assert rel_err(la, lc) < 2e-2          # the bf16 bound: cached values may round differently on the two paths
    del c
    first = int(np.argmax(la))
    steps = 24
    got, state = a.decode_fullvocab_sampled_run(first, 1.0, 1, steps)
    rng, tok, want = O.Rng(1), first, []
    for _ in range(steps):
        mx, sm = b.decode_token_block_stats_from_id(tok, 1.0, 0.0)
        blk = int(O.lib().orc_sample_block_from_stats(O.P(mx), O.P(sm), mx.size, rng.ref))
        bl = b.materialize_current_logits_block(blk, 0.0)
        tok = int(O.lib().orc_sample_block_logits(blk * 256, O.P(bl), bl.size, 1.0, rng.ref))
        want.append(tok)
    np.testing.assert_array_equal(got, np.array(want, np.uint32))
    assert state == rng.s.value
    assert a.len() == 1024 + steps


@pytest.mark.parametrize("wdt", [WeightDtype.FP8_E4M3, WeightDtype.INT4_G128])
def test_5b_quantised_workload_bf16_cache_512_token_prompt(w5b, wdt):
    """The quantised 5B workloads at their own shape: 512-token prompt, bf16 cache, greedy decode.
    Chunked prefill against token-step prefill (5e-2, the bound for 8-bit / 4-bit weights), a
    device-chained greedy run against the same steps taken one call at a time, and the step logits of
    the two models against each other."""
    cfg, w = w5b
    ids = synth.make_prompt(7, cfg.vocab, 512)
    a = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=KvDtype.BF16)
    b = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=KvDtype.BF16, flags=FLAG_PREFILL_STEPS)
    la, lb = a.prefill(ids), b.prefill(ids)
    assert rel_err(la, lb) < 5e-2
    first = int(np.argmax(la))
    run = a.decode_greedy_run(first, 16)
    a.set_len(512)
    tok, single = first, []
    for _ in range(16):
        tok = a.decode_token_argmax_from_id(tok)
        single.append(tok)
    np.testing.assert_array_equal(run, single)
    a.set_len(512)
    b.set_len(512)
    assert rel_err(a.decode_logits_from_id(first), b.decode_logits_from_id(first)) < 5e-2
