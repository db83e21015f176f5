"""The sampled token loops with the draw on the device (hipdec_decode_*_sampled_run*): the merge of
engine/src/decode.rs:218-253 and the draws of engine/src/inference.rs:823-921 done on the GPU must
give, token for token and with the same final RNG state, what the reference's loop gives when it
reads the candidates / block statistics back and draws on the host (inference.rs:586-625).

The draw needs exp() -- and the softcap of the merged candidates tanh() -- with the host C library's
bits.  The restatements the kernels use are checked here (a) on the host against libm: expf for
EVERY float <= 0 (the sampler's arguments are differences to a maximum, so never positive) and for
0..89, tanhf for all 2^32 floats; (b) against float64 exp / tanh; and (c) on the GPU against the
host evaluation through checksums over the same ranges."""
import ctypes as C
import ctypes.util

import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import engine as E
from rustane_amd import hipdec, synth
from rustane_amd.hipdec import Config, HipDecodeModel, KvDtype, WeightDtype

LIBM = C.CDLL(ctypes.util.find_library("m") or "libm.so.6")
LIBM.tanhf.restype = C.c_float
LIBM.tanhf.argtypes = [C.c_float]

NEG_FIRST, NEG_COUNT = 0x80000000, 0xFF800000 - 0x80000000 + 1      # -0.0 .. -inf
POS_FIRST, POS_COUNT = 0x00000000, 0x42B20000 + 1                   # +0.0 .. 89.0


# ------------------------------------------------------------------ the exponential (CPU)
EXPF, TANHF = hipdec.HOSTMATH_EXPF, hipdec.HOSTMATH_TANHF


def test_restated_expf_equals_libm_for_every_non_positive_float():
    assert hipdec.debug_hostmath_count_mismatch(EXPF, NEG_FIRST, NEG_COUNT, host_threads=8) == 0
    assert hipdec.debug_hostmath_count_mismatch(EXPF, POS_FIRST, POS_COUNT, host_threads=8) == 0


def test_library_probe_accepts_this_hosts_libm():
    # the sampled runs answer UNSUPPORTED where this is 0; here it must hold (the two exhaustive tests say so)
    assert hipdec.load_library().hipdec_debug_hostmath_probe() == 1


def test_restated_tanhf_equals_libm_for_every_float():
    assert hipdec.debug_hostmath_count_mismatch(TANHF, 0, 1 << 32, host_threads=8) == 0


def test_restated_tanhf_known_answers_and_float64_reference():
    x = np.array([0.0, -0.0, np.inf, -np.inf, 30.0, -30.0, 1e-20, 0.5, -2.0], np.float32)
    y = hipdec.debug_hostmath(TANHF, x)
    assert y[0] == 0.0 and np.signbit(y[1]) and y[2] == 1.0 and y[3] == -1.0 and y[4] == 1.0 and y[5] == -1.0
    assert y[6] == np.float32(1e-20)
    assert np.isnan(hipdec.debug_hostmath(TANHF, np.array([np.nan], np.float32))[0])
    rng = np.random.default_rng(6)
    x = np.concatenate([(rng.random(200000) * 2 - 1) * 12.0, (rng.random(100000) * 2 - 1) * 0.3]).astype(np.float32)
    y = hipdec.debug_hostmath(TANHF, x)
    want = np.tanh(x.astype(np.float64))
    ulp = np.spacing(np.abs(want).astype(np.float32)).astype(np.float64)
    assert np.all(np.abs(y.astype(np.float64) - want) <= 2.5 * ulp)         # the classic routine is good to ~2 ulp
    np.testing.assert_array_equal(hipdec.debug_hostmath(TANHF, -x), -y)    # odd


def test_restated_expf_known_answers_and_float64_reference():
    x = np.array([0.0, -0.0, -np.inf, np.inf, -104.0, -200.0, 89.0, 1.0, -1.0], np.float32)
    y = hipdec.debug_hostmath(EXPF, x)
    assert y[0] == 1.0 and y[1] == 1.0 and y[2] == 0.0 and np.isinf(y[3]) and y[4] == 0.0 and y[5] == 0.0
    assert np.isinf(y[6])                                            # exp(89) overflows float
    assert y[7] == np.float32(np.e) and y[8] == np.float32(1.0 / np.e)
    assert np.isnan(hipdec.debug_hostmath(EXPF, np.array([np.nan], np.float32))[0])
    rng = np.random.default_rng(5)
    x = np.concatenate([-rng.random(200000) * 104.0, rng.random(50000) * 88.0, -rng.random(50000) * 1e-3]).astype(np.float32)
    y = hipdec.debug_hostmath(EXPF, x)
    want = np.exp(x.astype(np.float64))
    # the C library documents 0.502 units in the last place for this algorithm
    ulp = np.maximum(np.spacing(want.astype(np.float32)).astype(np.float64), 2.0 ** -149)
    assert np.all(np.abs(y.astype(np.float64) - want) <= 0.503 * ulp)
    # subnormal results are produced, not flushed
    assert hipdec.debug_hostmath(EXPF, np.array([-100.0], np.float32))[0] == np.float32(np.exp(-100.0))


# ------------------------------------------------------------------ the exponential (GPU)
@pytest.mark.gpu
def test_device_expf_equals_host_expf_for_every_non_positive_float():
    for first, count in ((NEG_FIRST, NEG_COUNT), (POS_FIRST, POS_COUNT)):
        host = hipdec.debug_hostmath_checksum(EXPF, first, count, on_device=False, host_threads=16)
        dev = hipdec.debug_hostmath_checksum(EXPF, first, count, on_device=True)
        assert host == dev, (hex(first), hex(host), hex(dev))
    # element-wise on a sample, subnormal results and the special values included
    rng = np.random.default_rng(9)
    x = np.concatenate([-rng.random(100000) * 104.0, np.array([0.0, -0.0, -np.inf, -87.5, -88.0, -95.0, -103.9, -104.5])])
    x = x.astype(np.float32)
    np.testing.assert_array_equal(hipdec.debug_hostmath(EXPF, x, on_device=True).view(np.uint32), hipdec.debug_hostmath(EXPF, x).view(np.uint32))


@pytest.mark.gpu
def test_device_tanhf_equals_host_tanhf_for_every_float():
    host = hipdec.debug_hostmath_checksum(TANHF, 0, 1 << 32, on_device=False, host_threads=16)
    dev = hipdec.debug_hostmath_checksum(TANHF, 0, 1 << 32, on_device=True)
    assert host == dev, (hex(host), hex(dev))
    rng = np.random.default_rng(10)
    x = np.concatenate([(rng.random(100000) * 2 - 1) * 25.0, np.array([0.0, -0.0, np.inf, -np.inf, 1e-30, 0.3465, 1.0, 22.0])])
    x = x.astype(np.float32)
    np.testing.assert_array_equal(hipdec.debug_hostmath(TANHF, x, on_device=True).view(np.uint32),
                                  hipdec.debug_hostmath(TANHF, x).view(np.uint32))


# ------------------------------------------------------------------ the draw kernels on crafted inputs
def oracle_topk_draw(vals, idxs, k, T, seed, softcap=0.0):
    mv, mi = O.merge_topk(vals, idxs, k)
    mv = host_softcap(mv, softcap)
    rng = O.Rng(seed)
    tok = int(O.lib().orc_sample_topk_candidates(O.PU(mi), O.P(mv), mi.size, T, rng.ref)) if mi.size else 0
    if mi.size == 0:
        tok = 0                                   # inference.rs:829-831: no candidate, token 0, no draw
    return tok, rng.s.value


@pytest.mark.gpu
def test_topk_draw_kernel_on_crafted_candidate_lists():
    """Ties across blocks (lower index first), padded lists (index u32::MAX, value -inf), +inf / NaN
    values (dropped as the host merge drops them, decode.rs:229-231), fewer valid candidates than k,
    no valid candidate at all, weights that underflow: device merge + draw == oracle merge + draw."""
    MAXI = 0xFFFFFFFF
    rng = np.random.default_rng(3)
    cases = []
    for blocks, k in ((4, 8), (128, 8), (300, 32), (1024, 3), (1, 1), (2, 32)):
        vals = -np.sort(-rng.standard_normal((blocks, k)).astype(np.float32) * 3.0, axis=1)
        idxs = (np.arange(blocks)[:, None] * 256 + np.argsort(rng.random((blocks, 256)), axis=1)[:, :k]).astype(np.uint32)
        cases.append((vals.copy(), idxs.copy(), k))
        # ties: the same value at the head of several blocks
        v2, i2 = vals.copy(), idxs.copy()
        v2[:, 0] = np.float32(9.5)
        cases.append((v2, i2, k))
        # padding and non-finite entries
        v3, i3 = vals.copy(), idxs.copy()
        if k > 1:
            v3[::2, k // 2:] = -np.inf
            i3[::2, k // 2:] = MAXI
        v3[0, 0] = np.inf
        if blocks > 1:
            v3[1, 0] = np.nan
        cases.append((v3, i3, k))
        # hardly anything valid, and nothing valid
        v4, i4 = np.full_like(vals, -np.inf), np.full_like(idxs, MAXI)
        cases.append((v4.copy(), i4.copy(), k))
        v4[blocks - 1, 0], i4[blocks - 1, 0] = 1.25, 7
        cases.append((v4, i4, k))
        # a spread wide enough for zero and subnormal weights
        v5 = vals.copy()
        v5[0, 0] = 120.0
        cases.append((v5, idxs.copy(), k))
    seed = 1
    for n, (vals, idxs, k) in enumerate(cases):
        for T, cap in ((0.8, 0.0), (0.05, 0.0), (1.7, 2.0), (0.0, 0.0)):
            seed += 1
            got = hipdec.debug_sample_topk(vals.ravel(), idxs.ravel(), k, T, seed, softcap=cap)
            want = oracle_topk_draw(vals.ravel(), idxs.ravel(), k, T, seed, cap)
            assert got == want, (n, k, T, cap, got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("vocab", [1000, 256, 257, 8192])
def test_fullvocab_draw_kernel_on_crafted_logits(vocab):
    """Block draw from the statistics, token draw inside the block (the last block may be short):
    ordinary logits, blocks that are entirely -inf (weight 0), statistics with non-finite entries,
    and the all-non-finite case with its fallbacks (block 0, last maximal element)."""
    rng = np.random.default_rng(vocab)
    B = (vocab + 255) // 256
    base = (rng.standard_normal(vocab) * 4.0).astype(np.float32)
    variants = [base]
    v = base.copy(); v[:min(256, vocab)] = -np.inf; variants.append(v)          # a dead first block
    v = base.copy(); v[vocab - 1] = 50.0; variants.append(v)                    # nearly all mass in the last row
    v = np.full(vocab, -np.inf, np.float32); variants.append(v)                 # nothing finite anywhere
    seed = 10
    for n, lg in enumerate(variants):
        for T in (1.0, 0.3, 2.5):
            seed += 1
            inv_t = float(np.float32(1.0) / np.float32(T))
            with np.errstate(invalid="ignore"):
                mx, sm = O.block_stats(lg, inv_t, 0.0)
            for tweak in range(2):
                if tweak and B > 1:
                    mx, sm = mx.copy(), sm.copy()
                    sm[B // 2] = np.nan                                          # ignored block (inference.rs:861-866)
                    mx[0] = np.inf
                got = hipdec.debug_sample_fullvocab(lg, mx, sm, T, seed)
                r = O.Rng(seed)
                blk = int(O.lib().orc_sample_block_from_stats(O.P(mx), O.P(sm), mx.size, r.ref))
                bl = O.materialize_block(lg, blk, 0.0)
                tok = int(O.lib().orc_sample_block_logits(blk * 256, O.P(bl), bl.size, T, r.ref))
                assert got == (tok, r.s.value), (n, T, tweak, got, (tok, r.s.value))


# ------------------------------------------------------------------ runs against the host loop
def small_cfg(vocab=1000, seq=96):
    return Config.make(dim=256, hidden=640, heads=2, hd=128, seq=seq, nlayers=2, vocab=vocab)


def two_models(cfg, w, wd, kv, prompt):
    a = HipDecodeModel(cfg, w, weight_dtype=wd, kv_dtype=kv)
    b = HipDecodeModel(cfg, w, weight_dtype=wd, kv_dtype=kv)
    la = a.prefill(np.array(prompt, np.uint32))
    lb = b.prefill(np.array(prompt, np.uint32))
    np.testing.assert_array_equal(la, lb)
    return a, b, la


def host_softcap(v, cap):
    """decode.rs:155-159: cap * tanhf(v / cap) with the host C library's tanhf (float operations only)."""
    if cap <= 0.0:
        return v
    cap = np.float32(cap)
    t = np.array([LIBM.tanhf(C.c_float(float(np.float32(x) / cap))) for x in v], np.float32)
    return (cap * t).astype(np.float32)


def host_topk_loop(dev, tok, k, T, seed, steps, softcap=0.0):
    """inference.rs:586-599 with the oracle's merge and draw over the device's candidates."""
    rng = O.Rng(seed)
    out = []
    for _ in range(steps):
        vals, idxs = dev.decode_token_topk_from_id(tok, k)
        mv, mi = O.merge_topk(vals, idxs, k)
        mv = host_softcap(mv, softcap)
        tok = int(O.lib().orc_sample_topk_candidates(O.PU(mi), O.P(mv), mi.size, T, rng.ref))
        out.append(tok)
    return np.array(out, np.uint32), rng.s.value


def host_fullvocab_loop(dev, tok, T, softcap, seed, steps):
    """inference.rs:600-625 with the oracle's two draws over the device's statistics and block logits."""
    rng = O.Rng(seed)
    inv_t = np.float32(1.0) / max(np.float32(T), np.finfo(np.float32).tiny)
    out = []
    for _ in range(steps):
        mx, sm = dev.decode_token_block_stats_from_id(tok, float(inv_t), softcap)
        blk = int(O.lib().orc_sample_block_from_stats(O.P(mx), O.P(sm), mx.size, rng.ref))
        bl = dev.materialize_current_logits_block(blk, softcap)
        tok = int(O.lib().orc_sample_block_logits(blk * 256, O.P(bl), bl.size, T, rng.ref))
        out.append(tok)
    return np.array(out, np.uint32), rng.s.value


@pytest.mark.gpu
@pytest.mark.parametrize("wd,kv,vocab,k,T,softcap", [
    (WeightDtype.BF16, KvDtype.BF16, 1000, 8, 0.8, 0.0),      # last block holds 232 rows
    (WeightDtype.F32, KvDtype.F32, 8192, 4, 1.3, 0.0),
    (WeightDtype.FP8_E4M3, KvDtype.BF16, 320, 32, 0.5, 0.0),  # k > rows of the last block (64): padded lists
    (WeightDtype.BF16, KvDtype.F32, 1000, 1, 0.8, 0.0),       # one candidate: no draw, the state stays
    (WeightDtype.BF16, KvDtype.F32, 1000, 5, 0.0, 0.0),       # temperature 0: first candidate, no draw
    (WeightDtype.BF16, KvDtype.BF16, 1000, 8, 0.8, 3.0),      # softcap on the merged candidates (host tanhf)
    (WeightDtype.F32, KvDtype.F32, 8192, 16, 0.6, 0.75),
])
def test_topk_run_on_device_equals_host_loop(wd, kv, vocab, k, T, softcap):
    cfg = small_cfg(vocab)
    w = synth.make_weights(cfg, seed=13, std=0.08, round_bf16=True)
    a, b, lg = two_models(cfg, w, wd, kv, [3, 1, 4, 1, 5, 9, 2, 6])
    first = int(np.argmax(lg))
    steps, seed = 40, 0x1234567
    got, state = a.decode_topk_sampled_run(first, k, T, seed, steps, softcap=softcap)
    want, want_state = host_topk_loop(b, first, k, T, seed, steps, softcap)
    np.testing.assert_array_equal(got, want)
    assert state == want_state
    assert a.len() == b.len() == 8 + steps
    # a second run continues from where the first stopped, with the advanced state
    got2, state2 = a.decode_topk_sampled_run(int(got[-1]), k, T, state, 7, softcap=softcap)
    want2, want_state2 = host_topk_loop(b, int(want[-1]), k, T, want_state, 7, softcap)
    np.testing.assert_array_equal(got2, want2)
    assert state2 == want_state2
    if k > 1 and T > 0:
        assert state != seed and len(set(got.tolist())) > 1


@pytest.mark.gpu
@pytest.mark.parametrize("wd,kv,vocab,T,softcap", [
    (WeightDtype.BF16, KvDtype.BF16, 1000, 1.0, 0.0),
    (WeightDtype.F32, KvDtype.F32, 8192, 0.7, 0.0),
    (WeightDtype.BF16, KvDtype.F32, 320, 1.5, 2.5),      # softcap on the statistics and on the block
    (WeightDtype.INT4_G128, KvDtype.BF16, 1000, 1.0, 0.0),
])
def test_fullvocab_run_on_device_equals_host_loop(wd, kv, vocab, T, softcap):
    cfg = small_cfg(vocab)
    w = synth.make_weights(cfg, seed=17, std=0.08, round_bf16=True)
    a, b, lg = two_models(cfg, w, wd, kv, [2, 7, 1, 8, 2, 8, 1, 8])
    first = int(np.argmax(lg))
    steps, seed = 40, 99
    got, state = a.decode_fullvocab_sampled_run(first, T, seed, steps, softcap=softcap)
    want, want_state = host_fullvocab_loop(b, first, T, softcap, seed, steps)
    np.testing.assert_array_equal(got, want)
    assert state == want_state
    assert len(set(got.tolist())) > 4                     # two draws per token took place


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [1, 2, 3])      # eager launches, one kernel per product, both
@pytest.mark.parametrize("k", [6, 0])
def test_runs_on_device_without_graph_and_without_the_persistent_kernel(flags, k):
    """The draw kernels follow whatever produced the candidates / statistics: the same runs with the
    step launched eagerly (HIPDEC_FLAG_NO_GRAPH) and as one kernel per product (HIPDEC_FLAG_NO_MEGA)."""
    cfg = small_cfg(1000)
    w = synth.make_weights(cfg, seed=29, std=0.08, round_bf16=True)
    a = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16, flags=flags)
    b = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16, flags=flags)
    prompt = np.array([4, 8, 15, 16, 23, 42], np.uint32)
    lg = a.prefill(prompt)
    b.prefill(prompt)
    first, steps, seed = int(np.argmax(lg)), 20, 77
    if k > 0:
        got, state = a.decode_topk_sampled_run(first, k, 0.9, seed, steps, softcap=1.5)
        want, want_state = host_topk_loop(b, first, k, 0.9, seed, steps, 1.5)
    else:
        got, state = a.decode_fullvocab_sampled_run(first, 1.1, seed, steps)
        want, want_state = host_fullvocab_loop(b, first, 1.1, 0.0, seed, steps)
    np.testing.assert_array_equal(got, want)
    assert state == want_state and a.len() == b.len() == 6 + steps


@pytest.mark.gpu
@pytest.mark.parametrize("k,T,softcap", [(8, 0.8, 0.0), (0, 1.0, 0.0), (0, 0.9, 3.0), (6, 0.7, 2.0)])
def test_batched_run_on_device_equals_per_step_batch_calls(k, T, softcap):
    cfg = small_cfg(1000)
    w = synth.make_weights(cfg, seed=19, std=0.08, round_bf16=True)
    a, b, lg = two_models(cfg, w, WeightDtype.BF16, KvDtype.BF16, [5, 6, 7, 8, 9, 10, 11, 12, 13])
    R, steps = 5, 24
    first = np.argsort(lg)[::-1][:R].astype(np.uint32)    # rows start from different tokens
    seeds = np.arange(R, dtype=np.uint64) + np.uint64(21)
    a.batch_begin(R)
    b.batch_begin(R)
    if k > 0:
        got, states = a.decode_topk_sampled_run_batch(first, k, T, seeds, steps, softcap=softcap)
    else:
        got, states = a.decode_fullvocab_sampled_run_batch(first, T, seeds, steps, softcap=softcap)
    rngs = [O.Rng(int(s)) for s in seeds]
    cur = first.copy()
    inv_t = float(np.float32(1.0) / np.float32(T))
    for i in range(steps):
        nxt = np.empty(R, np.uint32)
        if k > 0:
            vals, idxs = b.decode_token_topk_from_ids_batch(cur, k)
            for r in range(R):
                mv, mi = O.merge_topk(vals[r], idxs[r], k)
                mv = host_softcap(mv, softcap)
                nxt[r] = O.lib().orc_sample_topk_candidates(O.PU(mi), O.P(mv), mi.size, T, rngs[r].ref)
        else:
            mx, sm = b.decode_token_block_stats_from_ids_batch(cur, inv_t, softcap)
            for r in range(R):
                mxr, smr = np.ascontiguousarray(mx[r]), np.ascontiguousarray(sm[r])
                blk = int(O.lib().orc_sample_block_from_stats(O.P(mxr), O.P(smr), mxr.size, rngs[r].ref))
                bl = b.materialize_current_logits_block_batch(r, blk, softcap)
                nxt[r] = O.lib().orc_sample_block_logits(blk * 256, O.P(bl), bl.size, T, rngs[r].ref)
        np.testing.assert_array_equal(got[i], nxt, err_msg="step %d" % i)
        cur = nxt
    np.testing.assert_array_equal(states, np.array([r.s.value for r in rngs], np.uint64))
    assert a.batch_steps() == b.batch_steps() == steps
    # the per-step calls continue an open batch after a run
    np.testing.assert_array_equal(a.decode_token_argmax_from_ids_batch(cur), b.decode_token_argmax_from_ids_batch(cur))
    a.batch_end()
    b.batch_end()


@pytest.mark.gpu
def test_run_argument_errors():
    cfg = small_cfg(1000, seq=32)
    w = synth.make_weights(cfg, seed=13, std=0.08, round_bf16=True)
    m = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32)
    m.prefill(np.array([1, 2, 3, 4], np.uint32))
    for bad_k in (0, 33):
        with pytest.raises(hipdec.HipDecodeError) as e:
            m.decode_topk_sampled_run(1, bad_k, 0.8, 1, 4)
        assert e.value.status == hipdec.ERR_ARG
    with pytest.raises(hipdec.HipDecodeError) as e:
        m.decode_fullvocab_sampled_run(1, 0.0, 1, 4)
    assert e.value.status == hipdec.ERR_ARG
    with pytest.raises(hipdec.HipDecodeError) as e:
        m.decode_topk_sampled_run(1, 8, 0.8, 1, 29)                 # 4 + 29 > seq
    assert e.value.status == hipdec.ERR_FULL
    with pytest.raises(hipdec.HipDecodeError) as e:
        m.decode_topk_sampled_run(5000, 8, 0.8, 1, 2)
    assert e.value.status == hipdec.ERR_ARG
    assert m.len() == 4                                             # nothing ran
    toks, st = m.decode_topk_sampled_run(1, 8, 0.8, 1, 0)           # zero steps: no-op
    assert toks.size == 0 and st == 1 and m.len() == 4
    toks, _ = m.decode_topk_sampled_run(1, 8, 0.8, 1, 28)           # exactly to the end of the cache
    assert toks.size == 28 and m.len() == 32


# ------------------------------------------------------------------ the session picks the device runs
@pytest.mark.gpu
@pytest.mark.parametrize("T,k,softcap,samples", [(0.8, 8, 0.0, 1), (1.0, 0, 0.0, 1), (1.0, 0, 2.5, 1), (0.8, 8, 0.0, 4),
                                                 (1.0, 0, 0.0, 3), (0.8, 4, 3.0, 2)])
def test_session_streams_are_the_same_with_device_and_host_draws(T, k, softcap, samples):
    cfg = small_cfg(1000, seq=64)
    prompt = [5, 6, 7, 8, 9, 10, 11, 12, 13]
    w = synth.make_weights(cfg, seed=31, std=0.08, round_bf16=True)
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=30, temperature=T, top_k=k, samples=samples, seed=21)
    dev = E.InferenceSession(cfg, w, prompt, softcap=softcap, weight_dtype=1).generate(req)
    host = E.InferenceSession(cfg, w, prompt, softcap=softcap, weight_dtype=1, flags=0x200).generate(req)
    assert len(dev.results) == len(host.results) == samples
    for a, b in zip(dev.results, host.results):
        np.testing.assert_array_equal(a.sampled, b.sampled)
        np.testing.assert_array_equal(a.generated, b.generated)
        assert a.seed == b.seed
    # a second request on the same session repeats the streams (prompt cache intact, RNG re-seeded)
    s = E.InferenceSession(cfg, w, prompt, softcap=softcap, weight_dtype=1)
    r1, r2 = s.generate(req), s.generate(req)
    for a, b in zip(r1.results, r2.results):
        np.testing.assert_array_equal(a.sampled, b.sampled)
