"""GPU parity of the multi-sample decode (hipdec_*_batch through the C ABI): every row of a batched
step must return what a sequential single-row run of that row returns (the reference draws its
samples one after the other, crates/engine/src/inference.rs:247-262, :561).  Each row is checked
against its own CPU oracle; tolerances as in crates/engine/tests/auto_kv_decode.rs:67-215."""
import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import synth
from rustane_amd.hipdec import (Config, HipDecodeModel, HipDecodeError, KvDtype, WeightDtype, ERR_ARG, ERR_FULL)

pytestmark = pytest.mark.gpu
ERR_UNSUPPORTED = 4


def rel_err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / max(np.abs(b).max(), 1e-30))


def setup(cfg, rows, n_prompt, wdt=WeightDtype.BF16, kvdt=KvDtype.F32, std=0.07, seed=17, round_bf16=True):
    w = synth.make_weights(cfg, seed=seed, std=std, round_bf16=round_bf16)
    wo = w
    if wdt == WeightDtype.FP8_E4M3:
        wo = O.dequantised_weights(cfg, w, "fp8")[0]
    if wdt == WeightDtype.INT4_G128:
        wo = O.dequantised_weights(cfg, w, "int4")[0]
    dev = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=kvdt)
    ids = synth.make_prompt(3, cfg.vocab, n_prompt)
    dev.prefill(ids, want_logits=False)
    orcs = []
    for _ in range(rows):
        o = O.Oracle(cfg, wo, kv_round_bf16=(kvdt == KvDtype.BF16))
        if n_prompt:
            o.forward_window(ids)
        orcs.append(o)
    return w, dev, orcs, ids


@pytest.mark.parametrize("rows,n_prompt", [(1, 9), (3, 20), (8, 40)])
def test_batched_logits_rows_match_sequential_oracles(rows, n_prompt):
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w, dev, orcs, ids = setup(cfg, rows, n_prompt)
    dev.batch_begin(rows)
    toks = np.array([(7 * r + 1) % cfg.vocab for r in range(rows)], np.uint32)
    for step in range(6):
        got = dev.decode_logits_from_ids_batch(toks)
        want = np.stack([orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)])
        for r in range(rows):
            assert rel_err(got[r], want[r]) < 1e-4, (step, r)
        # rows diverge: row r follows its own (r+1)-th best token
        toks = np.array([np.argsort(-want[r], kind="stable")[r % 4] for r in range(rows)], np.uint32)
    assert dev.batch_steps() == 6
    dev.batch_end()
    # the shared prefix is untouched: single-row decode continues from the prompt
    assert dev.len() == n_prompt
    fresh = O.Oracle(cfg, w)
    fresh.forward_window(ids)
    assert rel_err(dev.decode_logits_from_id(5), fresh.decode_logits_from_id(5)) < 1e-4


def test_batched_f32_weights():
    # (the reference's own format: its samples run one after the other; here they step together like the others)
    cfg = Config.make(dim=256, hidden=384, heads=4, hd=64, seq=64, nlayers=2, vocab=600, kv_heads=2)
    rows = 6
    w, dev, orcs, ids = setup(cfg, rows, 11, wdt=WeightDtype.F32, round_bf16=False)     # weights with all 24 bits in use
    dev.batch_begin(rows)
    toks = np.array([(13 * r + 2) % cfg.vocab for r in range(rows)], np.uint32)
    for step in range(5):
        got = dev.decode_logits_from_ids_batch(toks)
        want = np.stack([orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)])
        for r in range(rows):
            assert rel_err(got[r], want[r]) < 1e-4, (step, r)
        toks = np.array([np.argsort(-want[r], kind="stable")[r % 3] for r in range(rows)], np.uint32)
    dev.batch_end()


@pytest.mark.parametrize("rows", [5, 32])
def test_batched_4bit_weights_are_fp32_grade(rows):
    # 4-bit weights enter the few-row GEMM as exact integers and are scaled per 128-element group in fp32,
    # so every row is fp32-grade against the oracle run on the de-quantised weights.  3 and 9 scale groups
    # per weight row: the K splits and the four waves of a workgroup get uneven numbers of groups.
    cfg = Config.make(dim=384, hidden=1152, heads=3, hd=128, seq=64, nlayers=2, vocab=640)
    w, dev, orcs, ids = setup(cfg, rows, 12, wdt=WeightDtype.INT4_G128, std=0.05)
    dev.batch_begin(rows)
    toks = np.array([(11 * r + 3) % cfg.vocab for r in range(rows)], np.uint32)
    for step in range(4):
        got = dev.decode_logits_from_ids_batch(toks)
        want = np.stack([orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)])
        for r in range(rows):
            assert rel_err(got[r], want[r]) < 1e-4, (step, r)
        toks = np.array([np.argsort(-want[r], kind="stable")[r % 3] for r in range(rows)], np.uint32)
    dev.batch_end()


def test_batched_head_variants_match_oracle():
    cfg = Config.make(dim=256, hidden=384, heads=4, hd=64, seq=64, nlayers=2, vocab=600, kv_heads=2)
    rows = 4
    w, dev, orcs, ids = setup(cfg, rows, 12)
    dev.batch_begin(rows)
    toks = np.array([3, 50, 401, 599], np.uint32)
    # greedy
    got = dev.decode_token_argmax_from_ids_batch(toks)
    raw = [orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)]
    np.testing.assert_array_equal(got, [O.argmax_lower(x) for x in raw])
    toks = got
    # per-block top-k (value desc, index asc), ragged last block (600 = 2 * 256 + 88)
    k = 5
    vals, idxs = dev.decode_token_topk_from_ids_batch(toks, k)
    raw = [orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)]
    for r in range(rows):
        ov, oi = O.block_topk(raw[r], k)
        np.testing.assert_array_equal(idxs[r], oi)
        fin = np.isfinite(ov)
        assert rel_err(vals[r][fin], ov[fin]) < 1e-4
    toks = np.array([int(idxs[r][0]) for r in range(rows)], np.uint32)
    # block statistics + materialised block
    inv_t, cap = 1.0 / 0.8, 5.0
    mx, sm = dev.decode_token_block_stats_from_ids_batch(toks, inv_t, cap)
    raw = [orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)]
    for r in range(rows):
        omx, osm = O.block_stats(raw[r], inv_t, cap)
        assert rel_err(mx[r], omx) < 1e-4
        assert rel_err(sm[r], osm) < 1e-3
        for blk in (0, 2):
            got_b = dev.materialize_current_logits_block_batch(r, blk, cap)
            want_b = O.materialize_block(raw[r], blk, cap)
            assert got_b.size == want_b.size == (256 if blk == 0 else 88)
            assert rel_err(got_b, want_b) < 1e-4
    dev.batch_end()


def test_batched_bf16_cache_and_quantised_weights():
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=96, nlayers=2, vocab=512)
    for wdt in (WeightDtype.BF16, WeightDtype.FP8_E4M3, WeightDtype.INT4_G128):
        rows = 2
        w, dev, orcs, ids = setup(cfg, rows, 33, wdt=wdt, kvdt=KvDtype.BF16, std=0.05)
        dev.batch_begin(rows)
        toks = np.array([11, 300], np.uint32)
        for _ in range(4):
            got = dev.decode_logits_from_ids_batch(toks)
            want = np.stack([orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)])
            for r in range(rows):
                assert rel_err(got[r], want[r]) < 2e-3
            toks = np.array([O.argmax_lower(want[r]) for r in range(rows)], np.uint32)
        dev.batch_end()


def test_batched_error_codes():
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=12, nlayers=1, vocab=64)
    w = synth.make_weights(cfg, seed=2, std=0.05, round_bf16=True)
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16)
    with pytest.raises(HipDecodeError) as e:
        dev._rows = 2
        dev.decode_token_argmax_from_ids_batch([1, 2])
    assert e.value.status == ERR_ARG                      # no batch open
    with pytest.raises(HipDecodeError) as e:
        dev.batch_begin(33)
    assert e.value.status == ERR_ARG
    dev.prefill(synth.make_prompt(1, cfg.vocab, 10), want_logits=False)
    dev.batch_begin(2)
    with pytest.raises(HipDecodeError) as e:
        dev.decode_token_argmax_from_ids_batch([1, 64])
    assert e.value.status == ERR_ARG                      # token out of vocab
    dev.decode_token_argmax_from_ids_batch([1, 2])
    dev.decode_token_argmax_from_ids_batch([1, 2])
    with pytest.raises(HipDecodeError) as e:
        dev.decode_token_argmax_from_ids_batch([1, 2])
    assert e.value.status == ERR_FULL                     # 10 + 2 == seq
    dev.batch_end()
    # dimensions the few-row GEMM cannot tile (not multiples of 32): no multi-row step, the caller falls back
    odd = Config.make(dim=144, hidden=208, heads=1, hd=128, seq=12, nlayers=1, vocab=64)
    f32 = HipDecodeModel(odd, synth.make_weights(odd, seed=2, std=0.05), weight_dtype=WeightDtype.F32)
    with pytest.raises(HipDecodeError) as e:
        f32.batch_begin(2)
    assert e.value.status == ERR_UNSUPPORTED
