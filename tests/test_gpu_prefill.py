"""GPU parity of the chunked matrix-core prompt prefill (hipdec_prefill through the C ABI) against
the CPU oracle's full-window forward (crates/engine/src/full_model.rs:336-437) and against the
backend's own token-step prefill.  By default the prefill keeps activations fp32-grade (two bf16
parts; one fp16 number for 8-bit / 4-bit weights with a bf16 cache), so the fp32-cache tolerance is
the reference's 1e-4 on logits (crates/engine/tests/auto_kv_decode.rs:67-215); with a bf16 cache a
1-ulp difference can flip a cached value's rounding (2e-3)."""
import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import synth
from rustane_amd.hipdec import Config, HipDecodeModel, KvDtype, WeightDtype

pytestmark = pytest.mark.gpu

FLAG_PREFILL_STEPS = 4


def rel_err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / max(np.abs(b).max(), 1e-30))


def make(cfg, wdt=WeightDtype.BF16, kvdt=KvDtype.F32, std=0.06, seed=31, act=0, flags=0, round_bf16=True):
    w = synth.make_weights(cfg, seed=seed, std=std, round_bf16=round_bf16)
    wo = w
    if wdt == WeightDtype.FP8_E4M3:
        wo, _ = O.dequantised_weights(cfg, w, "fp8")
    if wdt == WeightDtype.INT4_G128:
        wo, _ = O.dequantised_weights(cfg, w, "int4")
    orc = O.Oracle(cfg, wo, kv_round_bf16=(kvdt == KvDtype.BF16), ffn_activation=act)
    dev = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=kvdt, ffn_activation=act, flags=flags)
    return w, orc, dev


def check_prefill_then_decode(cfg, n_prompt, tol, n_decode=4, **kw):
    w, orc, dev = make(cfg, **kw)
    ids = synth.make_prompt(3, cfg.vocab, n_prompt)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert dev.len() == n_prompt
    assert rel_err(lg_d, lg_o[0]) < tol
    # the caches the prefill wrote must carry the following cached steps
    tok = int(O.argmax_lower(lg_o[0]))
    for _ in range(n_decode):
        a = orc.decode_logits_from_id(tok)
        b = dev.decode_logits_from_id(tok)
        assert rel_err(b, a) < tol
        tok = int(O.argmax_lower(a))


@pytest.mark.parametrize("n_prompt", [8, 33, 70, 128])
def test_prefill_bf16_weights_f32_cache(n_prompt):
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=160, nlayers=2, vocab=320)
    check_prefill_then_decode(cfg, n_prompt, 1e-4)


@pytest.mark.parametrize("n_prompt", [8, 40, 97])
def test_prefill_f32_weights(n_prompt):
    # fp32 weights go through the few-row GEMM in chunks of 32 rows (40 = 32 + 8, 97 = 3 x 32 + 1 token step):
    # every weight as a (hi, lo) pair of bf16 numbers, three matrix instructions per product
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=160, nlayers=2, vocab=320)
    check_prefill_then_decode(cfg, n_prompt, 1e-4, wdt=WeightDtype.F32, round_bf16=False)   # weights with all 24 bits in use


def test_prefill_hd64_gqa_and_leaky_relu():
    cfg = Config.make(dim=256, hidden=384, heads=4, hd=64, seq=96, nlayers=3, vocab=512, kv_heads=2)
    check_prefill_then_decode(cfg, 45, 1e-4, act=1)


def test_prefill_bf16_cache():
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=200, nlayers=2, vocab=512)
    check_prefill_then_decode(cfg, 150, 2e-3, kvdt=KvDtype.BF16)


def test_prefill_fp8_weights():
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=128, nlayers=2, vocab=512)
    check_prefill_then_decode(cfg, 65, 2e-3, wdt=WeightDtype.FP8_E4M3, kvdt=KvDtype.BF16, std=0.05)


@pytest.mark.parametrize("n_prompt", [20, 65, 140])
def test_prefill_int4_weights(n_prompt):
    # 4-bit weights enter the matrix cores as exact integers and are scaled per group in fp32, so the
    # result is fp32-grade against the oracle run on the de-quantised weights
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=160, nlayers=2, vocab=512)
    check_prefill_then_decode(cfg, n_prompt, 1e-4, wdt=WeightDtype.INT4_G128, kvdt=KvDtype.F32, std=0.05)


@pytest.mark.parametrize("n_prompt", [5, 8, 13, 16, 27, 32])
def test_few_row_products_of_4bit_weights(n_prompt):
    # prompts of at most 32 rows go through the few-row GEMM of 4-bit weights: hi and lo parts in one operand tile
    # up to 8 rows, one and two row tiles above; reductions of 3 groups (dim 384: the short scale path), 4 (q_dim 512)
    # and 9 (hidden 1152: splits of 4 + 4 + 1 groups, a round that ends early)
    cfg = Config.make(dim=384, hidden=1152, heads=4, hd=128, seq=64, nlayers=3, vocab=768, kv_heads=2)
    check_prefill_then_decode(cfg, n_prompt, 1e-4, wdt=WeightDtype.INT4_G128, kvdt=KvDtype.F32, std=0.05)


@pytest.mark.parametrize("n_prompt", [6, 8, 14, 31])
def test_few_row_products_of_e4m3_weights(n_prompt):
    # prompts of at most 32 rows of an e4m3 model go through the few-row GEMM written for that format (reductions
    # that are multiples of 64: dim 384, q_dim 512, hidden 1152 = 18 blocks, i.e. rounds and splits that end early)
    cfg = Config.make(dim=384, hidden=1152, heads=4, hd=128, seq=64, nlayers=3, vocab=768, kv_heads=2)
    check_prefill_then_decode(cfg, n_prompt, 1e-4, wdt=WeightDtype.FP8_E4M3, kvdt=KvDtype.F32, std=0.05)


def test_prefill_int4_matches_token_step_prefill():
    cfg = Config.make(dim=384, hidden=1152, heads=3, hd=128, seq=200, nlayers=3, vocab=1024)
    w = synth.make_weights(cfg, seed=5, std=0.06, round_bf16=True)
    ids = synth.make_prompt(4, cfg.vocab, 150)
    a = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.INT4_G128, kv_dtype=KvDtype.BF16)
    b = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.INT4_G128, kv_dtype=KvDtype.BF16, flags=FLAG_PREFILL_STEPS)
    la, lb = a.prefill(ids), b.prefill(ids)
    assert rel_err(la, lb) < 2e-3                 # bf16 cache: a 1-ulp difference can flip a cached rounding
    ta = a.decode_greedy_run(int(np.argmax(la)), 16)
    tb = b.decode_greedy_run(int(np.argmax(lb)), 16)
    np.testing.assert_array_equal(ta, tb)


def test_prefill_in_two_calls_equals_one():
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=160, nlayers=2, vocab=320)
    w, orc, dev = make(cfg)
    ids = synth.make_prompt(9, cfg.vocab, 90)
    lg_o, _, _ = orc.forward_window(ids)
    dev.prefill(ids[:50], want_logits=False)
    lg_d = dev.prefill(ids[50:])
    assert dev.len() == 90
    assert rel_err(lg_d, lg_o[0]) < 1e-4


def test_chunked_prefill_matches_token_step_prefill():
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=256, nlayers=3, vocab=1024)
    w = synth.make_weights(cfg, seed=5, std=0.06, round_bf16=True)
    ids = synth.make_prompt(4, cfg.vocab, 130)
    a = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32)
    b = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32, flags=FLAG_PREFILL_STEPS)
    la, lb = a.prefill(ids), b.prefill(ids)
    assert rel_err(la, lb) < 2e-5
    ta = a.decode_greedy_run(int(np.argmax(la)), 16)
    tb = b.decode_greedy_run(int(np.argmax(lb)), 16)
    np.testing.assert_array_equal(ta, tb)


def test_prefill_longer_than_one_chunk_and_empty_prefill():
    # 1100 rows = one full 1024-row chunk + a 76-row chunk whose attention starts at position 1024
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=1200, nlayers=2, vocab=320)
    w, orc, dev = make(cfg)
    ids = synth.make_prompt(11, cfg.vocab, 1100)
    lg_o, _, _ = orc.forward_window(ids)
    dev.prefill(ids[:0], want_logits=False)            # nothing to do, nothing changes
    assert dev.len() == 0
    lg_d = dev.prefill(ids)
    assert dev.len() == 1100
    assert rel_err(lg_d, lg_o[0]) < 1e-4
    tok = int(O.argmax_lower(lg_o[0]))
    assert rel_err(dev.decode_logits_from_id(tok), orc.decode_logits_from_id(tok)) < 1e-4


FLAG_PREFILL_BF16_ACT, FLAG_PREFILL_F16_ACT, FLAG_PREFILL_PAIR_ACT = 8, 16, 32


@pytest.mark.parametrize("flag,bound", [(FLAG_PREFILL_BF16_ACT, 2e-2), (FLAG_PREFILL_F16_ACT, 3e-3)])
@pytest.mark.parametrize("wdt,n_prompt", [(WeightDtype.FP8_E4M3, 140), (WeightDtype.INT4_G128, 140), (WeightDtype.BF16, 70)])
def test_prefill_with_single_number_activations(wdt, n_prompt, flag, bound):
    """HIPDEC_FLAG_PREFILL_BF16_ACT / _F16_ACT: the prefill GEMMs multiply the weights by the activations
    rounded to ONE bf16 (8 mantissa bits) or fp16 (11 bits) number instead of the (hi, lo) bf16 pair, i.e.
    half the matrix-core work.  Stated bounds against the oracle: 5e-2 of the largest logit for bf16, the
    bf16-cache tolerance of this file for fp16; what is measured on this 3-layer model is asserted (2e-2,
    3e-3), the token the prompt logits elect is the same as with the pair, the caches that prefill leaves
    carry the following cached steps (whose own arithmetic is unchanged) to the same bound, and the mode
    can be switched on a live model.  (fp16 is what an 8-bit / 4-bit model with a bf16 cache uses unless told
    otherwise; the pair is requested with its own flag here.)"""
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=192, nlayers=3, vocab=512)
    kw = dict(wdt=wdt, kvdt=KvDtype.BF16, std=0.05)
    w, orc, dev = make(cfg, flags=flag, **kw)
    _, _, ref = make(cfg, flags=FLAG_PREFILL_PAIR_ACT, **kw)
    ids = synth.make_prompt(3, cfg.vocab, n_prompt)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d, lg_r = dev.prefill(ids), ref.prefill(ids)
    err, err_pair = rel_err(lg_d, lg_o[0]), rel_err(lg_r, lg_o[0])
    print("single-number activations (flag %d): %.2e of the largest logit against the oracle (pair: %.2e)" % (flag, err, err_pair))
    assert err_pair < 3e-3 and err < bound
    if flag == FLAG_PREFILL_BF16_ACT:
        assert err > err_pair
    assert int(np.argmax(lg_d)) == int(np.argmax(lg_r)) == int(O.argmax_lower(lg_o[0]))
    tok = int(O.argmax_lower(lg_o[0]))
    for _ in range(4):
        a = orc.decode_logits_from_id(tok)
        assert rel_err(dev.decode_logits_from_id(tok), a) < bound
        tok = int(O.argmax_lower(a))
    # the same switch at run time: the pair model in this mode gives this model's logits bit for bit, and back
    ref.set_prefill_activations(1 if flag == FLAG_PREFILL_BF16_ACT else 2)
    ref.set_len(0)
    np.testing.assert_array_equal(ref.prefill(ids), lg_d)
    ref.set_prefill_activations(0)
    ref.set_len(0)
    np.testing.assert_array_equal(ref.prefill(ids), lg_r)
    # mode 3: the pair into the q/k/v and output projections, single bf16 numbers into the two feed-forward products
    ref.set_prefill_activations(3)
    ref.set_len(0)
    lg_m = ref.prefill(ids)
    assert rel_err(lg_m, lg_r) <= max(rel_err(lg_d, lg_r), 1e-6) * 1.5 + 1e-4 if flag == FLAG_PREFILL_BF16_ACT else True
    ref.set_prefill_activations(0)
    with pytest.raises(Exception):
        ref.set_prefill_activations(4)
