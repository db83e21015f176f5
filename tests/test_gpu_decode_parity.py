"""GPU parity: the HIP decode backend, called through the C ABI, against the CPU oracle on the
same seeded weights and prompts.  Shapes and tolerances follow the reference's own decode parity
tests (crates/engine/tests/auto_kv_decode.rs:7-28, :67-215): exact greedy ids, exact top-k ids,
1e-4 on logits, 1e-3 on block sums."""
import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import synth
from rustane_amd.hipdec import (Config, HipDecodeModel, HipDecodeError, KvDtype, WeightDtype, ERR_ARG, ERR_FULL)

pytestmark = pytest.mark.gpu


def tiny_cfg(vocab=64):
    # auto_kv_decode.rs:7-21 (vocab 64) and :23-28 (vocab 320 = two head blocks)
    return Config.make(dim=256, hidden=640, heads=2, hd=128, seq=64, nlayers=2, vocab=vocab)


def rel_err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / max(np.abs(b).max(), 1e-30))


def pair(cfg, seed=11, std=0.02, wdt=WeightDtype.F32, kvdt=KvDtype.F32, flags=0, act=0):
    w = synth.make_weights(cfg, seed=seed, std=std, round_bf16=(wdt != WeightDtype.F32))
    orc = O.Oracle(cfg, w, kv_round_bf16=(kvdt == KvDtype.BF16), ffn_activation=act)
    dev = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=kvdt, flags=flags, ffn_activation=act)
    return w, orc, dev


@pytest.mark.parametrize("std", [0.02, 0.08])
@pytest.mark.parametrize("flags", [0, 1])
def test_prefill_then_logits_match_oracle_fp32(std, flags):
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg, std=std, flags=flags)
    ids = np.array([1, 2, 3, 4, 5], np.uint32)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert dev.len() == 5 and orc.len() == 5
    assert rel_err(lg_d, lg_o[0]) < 1e-4
    tok = int(O.argmax_lower(lg_o[0]))
    for _ in range(6):
        a = orc.decode_logits_from_id(tok)
        b = dev.decode_logits_from_id(tok)
        assert rel_err(b, a) < 1e-4
        assert O.argmax_lower(b) == O.argmax_lower(a)
        tok = int(O.argmax_lower(a))
    assert dev.len() == 11


def test_seeded_cache_greedy_tokens_match_window_forward():
    # auto_kv_decode.rs:67-134: prompt through the full-window forward, caches handed over
    # channel-first, then three cached steps against re-running the window.
    cfg = tiny_cfg(64)
    w, orc, dev = pair(cfg, std=0.08)
    generated = [1, 2, 3]
    lg, k_cf, v_cf = orc.forward_window(np.array(generated, np.uint32), want_caches=True)
    dev.set_len(len(generated))
    for l in range(cfg.nlayers):
        dev.seed_layer_cache_from_channel_first(l, len(generated), k_cf[l], v_cf[l])
    nxt = int(O.argmax_last(lg[0]))
    generated.append(nxt)
    for _ in range(3):
        cached_next = dev.decode_token_argmax_from_id(nxt)
        lg, _, _ = O.Oracle(cfg, w).forward_window(np.array(generated, np.uint32))
        assert cached_next == int(O.argmax_lower(lg[0]))
        nxt = cached_next
        generated.append(nxt)


def test_decode_token_variants_match_oracle():
    cfg = tiny_cfg(64)
    w, orc, dev = pair(cfg, std=0.08)
    for tok in (3, 9):
        a = orc.decode_token_from_id(tok)
        b = dev.decode_token_from_id(tok)
        assert rel_err(b, a) < 1e-5
    x_in = synth.synth_normal(99, 7, cfg.dim, std=0.3)
    a = orc.decode_token(x_in)
    b = dev.decode_token(x_in)
    assert rel_err(b, a) < 1e-5
    # argmax from a caller-supplied residual stream
    orc_x = orc.decode_token(x_in)
    xf = orc_x / np.sqrt((orc_x.astype(np.float64) ** 2).mean() + 1e-5)
    want = int(np.argmax(w["embed"].reshape(cfg.vocab, cfg.dim).astype(np.float64) @ xf))
    got = dev.decode_token_argmax(x_in)
    assert got == want
    assert dev.len() == 4


def test_topk_candidates_match_oracle():
    # auto_kv_decode.rs:136-173 (vocab 320: the second block is ragged)
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg, std=0.08)
    ids = np.array([1, 2, 3], np.uint32)
    orc.forward_window(ids)
    dev.prefill(ids, want_logits=False)
    for k in (1, 4, 32):
        raw = orc.decode_logits_from_id(7)
        vals, idxs = dev.decode_token_topk_from_id(7, k)
        ov, oi = O.block_topk(raw, k)
        assert vals.size == dev.blocks * k
        np.testing.assert_array_equal(idxs, oi)
        finite = np.isfinite(ov)
        assert rel_err(vals[finite], ov[finite]) < 1e-4
        assert np.all(np.isneginf(vals[~finite]))
        mv, mi = O.merge_topk(vals, idxs, k)
        order = np.lexsort((np.arange(raw.size), -raw))[:k]
        np.testing.assert_array_equal(mi, order.astype(np.uint32))


def test_block_stats_and_materialize_match_oracle():
    # auto_kv_decode.rs:175-215
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg, std=0.08)
    ids = np.array([1, 2, 3, 4], np.uint32)
    orc.forward_window(ids)
    dev.prefill(ids, want_logits=False)
    for temperature, softcap in ((0.8, 0.0), (1.0, 5.0)):
        raw = orc.decode_logits_from_id(5)
        mx, sm = dev.decode_token_block_stats_from_id(5, 1.0 / temperature, softcap)
        omx, osm = O.block_stats(raw, 1.0 / temperature, softcap)
        assert np.abs(mx - omx).max() < 1e-4
        assert np.abs(sm - osm).max() < 1e-3
        blk = dev.materialize_current_logits_block(1, softcap)
        want = O.materialize_block(raw, 1, softcap)
        assert blk.size == 64
        assert np.abs(blk - want).max() < 1e-4
    assert dev.len() == 6          # materialise does not advance


def test_greedy_run_equals_single_steps_and_oracle():
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg, std=0.08)
    _, _, dev2 = pair(cfg, std=0.08)
    ids = np.array([5, 6, 7], np.uint32)
    lg, _, _ = orc.forward_window(ids)
    dev.prefill(ids, want_logits=False)
    dev2.prefill(ids, want_logits=False)
    first = int(O.argmax_last(lg[0]))
    run = dev.decode_greedy_run(first, 20)
    cur, singles = first, []
    for _ in range(20):
        cur = dev2.decode_token_argmax_from_id(cur)
        singles.append(cur)
    np.testing.assert_array_equal(run, np.array(singles, np.uint32))
    sampled, _ = orc.run_cached_sample(ids, lg[0], 21)
    np.testing.assert_array_equal(run, sampled[1:])
    assert dev.len() == 23 and dev2.len() == 23


def test_c1_tiny_greedy_32_steps_identical_and_logits_1e4():
    # configuration 1: dim 512, 8 layers, 8 heads x 64, hidden 1536, vocab 8192, seq 512, fp32
    cfg = synth.config_c1()
    w, orc, dev = pair(cfg, seed=1234)
    prompt = synth.make_prompt(7, cfg.vocab, 4)
    lg_o, _, _ = orc.forward_window(prompt)
    lg_d = dev.prefill(prompt)
    assert rel_err(lg_d, lg_o[0]) < 1e-4
    sampled, _ = orc.run_cached_sample(prompt, lg_o[0], 32)
    got = dev.decode_greedy_run(int(sampled[0]), 31)
    np.testing.assert_array_equal(got, sampled[1:])
    a = orc.decode_logits_from_id(int(sampled[-1]))
    b = dev.decode_logits_from_id(int(sampled[-1]))
    assert rel_err(b, a) < 1e-4


def test_c1_shape_nondegenerate_stream():
    # same shape with wider weights so that the greedy stream is not a fixed point
    cfg = synth.config_c1()
    w, orc, dev = pair(cfg, seed=77, std=0.07)
    prompt = synth.make_prompt(9, cfg.vocab, 6)
    lg_o, _, _ = orc.forward_window(prompt)
    lg_d = dev.prefill(prompt)
    assert rel_err(lg_d, lg_o[0]) < 1e-4
    sampled, _ = orc.run_cached_sample(prompt, lg_o[0], 48)
    assert len(set(sampled.tolist())) > 8
    got = dev.decode_greedy_run(int(sampled[0]), 47)
    np.testing.assert_array_equal(got, sampled[1:])


@pytest.mark.parametrize("kvdt", [KvDtype.F32, KvDtype.BF16])
def test_bf16_weights_match_oracle(kvdt):
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=128, nlayers=3, vocab=1000)
    w, orc, dev = pair(cfg, seed=3, std=0.06, wdt=WeightDtype.BF16, kvdt=kvdt)
    ids = synth.make_prompt(3, cfg.vocab, 9)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert rel_err(lg_d, lg_o[0]) < 2e-2       # north-star bf16 bound
    # fp32 accumulation over bf16-exact weights agrees to round-off; with a bf16 cache a 1-ulp
    # difference upstream can flip the rounding of a cached value, which is a 2^-8 step
    assert rel_err(lg_d, lg_o[0]) < (1e-4 if kvdt == KvDtype.F32 else 2e-3)
    sampled, _ = orc.run_cached_sample(ids, lg_o[0], 40)
    got = dev.decode_greedy_run(int(sampled[0]), 39)
    np.testing.assert_array_equal(got, sampled[1:])
    k = orc.kcache(1)[: dev.len()]
    assert np.isfinite(k).all()


def test_leaky_relu_sq_activation():
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg, std=0.08, act=1)
    ids = np.array([1, 2, 3], np.uint32)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert rel_err(lg_d, lg_o[0]) < 1e-4


@pytest.mark.parametrize("wdt,which_tol", [(WeightDtype.FP8_E4M3, 5e-2), (WeightDtype.INT4_G128, 5e-2)])
def test_quantised_weights_bit_exact_and_logits(wdt, which_tol):
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=64, nlayers=2, vocab=512)
    w = synth.make_weights(cfg, seed=21, std=0.05, round_bf16=True)
    dev = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=KvDtype.BF16)
    L = O.lib()
    D, Q, KV, H = cfg.dim, cfg.q_dim, cfg.kv_dim, cfg.hidden

    def out_major(a, rows_in, cols_in, transpose):
        a = O.f32(a).reshape(rows_in, cols_in)
        return np.ascontiguousarray(a.T) if transpose else a

    def dq(m):
        m = np.ascontiguousarray(m, np.float32)
        out = np.empty_like(m)
        if wdt == WeightDtype.FP8_E4M3:
            L.orc_quant_fp8_rows(O.P(m), m.shape[0], m.shape[1], None, None, O.P(out))
        else:
            L.orc_quant_int4_g128(O.P(m), m.shape[0], m.shape[1], None, None, O.P(out))
        return out

    wq_dq = {"embed": w["embed"], "gamma_final": w["gamma_final"], "layers": []}
    for l, lw in enumerate(w["layers"]):
        mats = {n: dq(out_major(lw[n], *shape)) for n, shape in
                dict(wq=(D, Q, True), wk=(D, KV, True), wv=(D, KV, True), wo=(Q, D, True), w1=(D, H, True),
                     w3=(D, H, True), w2=(D, H, False)).items()}
        # stored weights, de-quantised on the device, must equal the oracle's bit for bit
        qkv = dev.export_weight(l, 0)
        np.testing.assert_array_equal(qkv, np.concatenate([mats["wq"], mats["wk"], mats["wv"]], 0))
        np.testing.assert_array_equal(dev.export_weight(l, 1), mats["wo"])
        w13 = dev.export_weight(l, 2)
        np.testing.assert_array_equal(w13[0::2], mats["w1"])
        np.testing.assert_array_equal(w13[1::2], mats["w3"])
        np.testing.assert_array_equal(dev.export_weight(l, 3), mats["w2"])
        lay = {n: np.ascontiguousarray(mats[n].T).ravel() for n in ("wq", "wk", "wv", "wo", "w1", "w3")}
        lay["w2"] = mats["w2"].ravel()
        lay["gamma1"], lay["gamma2"] = lw["gamma1"], lw["gamma2"]
        wq_dq["layers"].append(lay)
    np.testing.assert_array_equal(dev.export_weight(0, 4).ravel(), w["embed"])
    orc = O.Oracle(cfg, wq_dq, kv_round_bf16=True)
    ids = synth.make_prompt(5, cfg.vocab, 6)
    lg_o, _, _ = orc.forward_window(ids)
    lg_d = dev.prefill(ids)
    assert rel_err(lg_d, lg_o[0]) < which_tol
    assert rel_err(lg_d, lg_o[0]) < 2e-3       # bf16 cache: a 1-ulp difference can flip a cached value's rounding
    sampled, _ = orc.run_cached_sample(ids, lg_o[0], 24)
    got = dev.decode_greedy_run(int(sampled[0]), 23)
    np.testing.assert_array_equal(got, sampled[1:])


def test_error_codes_replace_panics():
    # crates/metal-decode/src/lib.rs:242-245, :277-280, :392-405, :452-453, :495, :501
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg)
    with pytest.raises(HipDecodeError) as e:
        dev.decode_token_argmax_from_id(cfg.vocab)
    assert e.value.status == ERR_ARG
    for k in (0, 33):
        with pytest.raises(HipDecodeError) as e:
            dev.decode_token_topk_from_id(1, k)
        assert e.value.status == ERR_ARG
    with pytest.raises(HipDecodeError) as e:
        dev.decode_token_topk_from_id(1, 4, cap=7)
    assert e.value.status == ERR_ARG
    with pytest.raises(HipDecodeError) as e:
        dev.decode_token_block_stats_from_id(1, 1.0, 0.0, cap=1)
    assert e.value.status == ERR_ARG
    with pytest.raises(HipDecodeError) as e:
        dev.materialize_current_logits_block(2, 0.0)
    assert e.value.status == ERR_ARG
    with pytest.raises(HipDecodeError) as e:
        dev.materialize_current_logits_block(1, 0.0, cap=10)
    assert e.value.status == ERR_ARG
    assert dev.len() == 0
    dev.set_len(10_000)
    assert dev.len() == cfg.seq            # set_len clamps, lib.rs:213-215
    with pytest.raises(HipDecodeError) as e:
        dev.decode_token_argmax_from_id(1)
    assert e.value.status == ERR_FULL
    dev.set_len(cfg.seq - 1)
    dev.decode_token_argmax_from_id(1)     # the last slot is usable
    assert dev.len() == cfg.seq


@pytest.mark.parametrize("wdt,kvdt", [(WeightDtype.F32, KvDtype.F32), (WeightDtype.BF16, KvDtype.BF16),
                                      (WeightDtype.FP8_E4M3, KvDtype.BF16)])
def test_graph_replay_equals_eager_launch_and_runs_repeat_bit_for_bit(wdt, kvdt):
    """The reference checks its reordered schedules against the straightforward ones with tolerance 0.0
    (its auto_*.rs tests).  Here: the captured-graph step against eager launches of the same kernels,
    and a run against its own repetition -- every reduction has a fixed order, so the bits must agree.
    Covers single steps, the chained greedy run and the multi-row step."""
    cfg = tiny_cfg(1000)
    w = synth.make_weights(cfg, seed=23, std=0.08, round_bf16=True)
    graph = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=kvdt)
    eager = HipDecodeModel(cfg, w, weight_dtype=wdt, kv_dtype=kvdt, flags=1)
    ids = np.array([7, 1, 9, 4, 4, 2, 8, 3, 5, 6], np.uint32)

    def run(dev):
        dev.set_len(0)
        out = [dev.prefill(ids)]
        tok = int(np.argmax(out[0]))
        for _ in range(5):
            out.append(dev.decode_logits_from_id(tok))
            tok = int(np.argmax(out[-1]))
        out.append(dev.decode_greedy_run(tok, 6).astype(np.float32))
        vals, idxs = dev.decode_token_topk_from_id(int(out[-1][-1]), 4)
        out += [vals, idxs.astype(np.float32)]
        if wdt != WeightDtype.F32:                               # the multi-row step needs 16-bit or 8-bit weights
            dev.batch_begin(3)
            toks = np.array([1, 2, 3], np.uint32)
            for _ in range(3):
                lg = dev.decode_logits_from_ids_batch(toks)
                out.append(lg)
                toks = np.argmax(lg, axis=1).astype(np.uint32)
            dev.batch_end()
        return out

    a, b, c = run(graph), run(eager), run(graph)
    assert len(a) == len(b) == len(c)
    for x, y, z in zip(a, b, c):
        np.testing.assert_array_equal(x.view(np.uint32), y.view(np.uint32))
        np.testing.assert_array_equal(x.view(np.uint32), z.view(np.uint32))


def _free_device_bytes():
    import ctypes as C
    rt = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert rt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


@pytest.mark.gpu
def test_models_sharing_one_copy_of_the_weights():
    """hipdec_create_shared: a second model on the first one's device weights (the reference uploads per
    Model::new, crates/metal-decode/src/lib.rs:147-207).  Both give the logits of an independently created
    model, bit for bit, with their own caches and positions; the second costs caches and workspaces, not
    weights; the weights outlive the model that uploaded them."""
    cfg = Config.make(dim=512, hidden=2048, heads=4, hd=128, seq=64, nlayers=4, vocab=4096)
    w = synth.make_weights(cfg, seed=21, std=0.06, round_bf16=True)
    weight_bytes = 2 * (cfg.nlayers * (4 * cfg.dim * cfg.dim + 3 * cfg.dim * cfg.hidden) + cfg.vocab * cfg.dim)
    ids_a = synth.make_prompt(5, cfg.vocab, 12)
    ids_b = synth.make_prompt(6, cfg.vocab, 20)
    ref = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32)
    want_a, want_b = ref.prefill(ids_a), None
    ref.set_len(0)
    want_b = ref.prefill(ids_b)
    ref.close()

    before = _free_device_bytes()
    base = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32)
    after_base = _free_device_bytes()
    twin = base.create_shared(kv_dtype=KvDtype.F32)
    after_twin = _free_device_bytes()
    assert before - after_base >= weight_bytes                         # the first model holds the weights ...
    assert after_base - after_twin < weight_bytes // 4                 # ... the second one only caches and workspaces
    np.testing.assert_array_equal(base.prefill(ids_a), want_a)
    np.testing.assert_array_equal(twin.prefill(ids_b), want_b)         # interleaved use, separate caches
    assert (base.len(), twin.len()) == (12, 20)
    ta, tb = int(np.argmax(want_a)), int(np.argmax(want_b))
    la, lb = base.decode_logits_from_id(ta), twin.decode_logits_from_id(tb)
    base.close()                                                       # the uploader goes first
    ref2 = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32)
    ref2.prefill(ids_b)
    np.testing.assert_array_equal(ref2.decode_logits_from_id(tb), lb)
    np.testing.assert_array_equal(twin.decode_greedy_run(int(np.argmax(lb)), 8), ref2.decode_greedy_run(int(np.argmax(lb)), 8))
    ref2.set_len(0)
    ref2.prefill(ids_a)
    np.testing.assert_array_equal(ref2.decode_logits_from_id(ta), la)
    # a bf16 cache on the same weights
    twin16 = twin.create_shared(kv_dtype=KvDtype.BF16)
    solo16 = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.BF16)
    np.testing.assert_array_equal(twin16.prefill(ids_a), solo16.prefill(ids_a))
    twin.close()
    np.testing.assert_array_equal(twin16.decode_logits_from_id(ta), solo16.decode_logits_from_id(ta))


def test_a_wait_that_gives_up_leaves_the_model_on_the_one_kernel_per_product_path():
    """The persistent step kernel bounds every wait on another workgroup.  With the bound set to zero polls
    (a test hook; every kernel still exits normally) the first stale poll gives up: the call reports
    HIPDEC_ERR_HIP, the length is unchanged, and the model takes the one-kernel-per-product path from then
    on -- the retried step and the steps after it against the oracle."""
    from rustane_amd import hipdec
    from rustane_amd.hipdec import ERR_HIP
    cfg = tiny_cfg(320)
    w, orc, dev = pair(cfg, std=0.08)
    ids = np.array([4, 9, 2, 7, 1], np.uint32)
    orc.forward_window(ids)
    dev.prefill(ids, want_logits=False)
    tok, failed = 3, False
    hipdec.set_spin_limit(0, 0)
    try:
        for _ in range(8):                       # (a step whose polls all find fresh values would pass: try a few)
            n0 = dev.len()
            try:
                got = dev.decode_logits_from_id(tok)
            except HipDecodeError as e:
                assert e.status == ERR_HIP and "timed out" in str(e)
                assert dev.len() == n0
                failed = True
                break
            want = orc.decode_logits_from_id(tok)
            assert rel_err(got, want) < 1e-4
            tok = int(O.argmax_lower(want))
    finally:
        hipdec.set_spin_limit()
    assert failed, "no wait gave up with a zero poll limit"
    for _ in range(5):
        want = orc.decode_logits_from_id(tok)
        got = dev.decode_logits_from_id(tok)
        assert rel_err(got, want) < 1e-4
        assert dev.decode_token_argmax_from_id(int(O.argmax_lower(want))) == int(O.argmax_lower(orc.decode_logits_from_id(int(O.argmax_lower(want)))))
        tok = int(O.argmax_lower(want))


# ---- the short-phase form of the persistent step kernel (hipdec_lean.h): bf16 weights, reduction lengths multiples of 512
LEAN_SHAPES = [
    # dim 512: one chunk per row of the even phases; hd 128, fp32 cache
    (dict(dim=512, hidden=1024, heads=4, hd=128, seq=96, nlayers=3, vocab=320), KvDtype.F32, 0, 1e-4),
    # grouped key/value heads of 64, squared leaky ReLU, bf16 cache, an odd layer count
    (dict(dim=512, hidden=512, heads=8, hd=64, seq=96, nlayers=3, vocab=600, kv_heads=4), KvDtype.BF16, 1, 2e-3),
    # dim 1536 (three chunks per row, the 600M-class width), down projection of 2048
    (dict(dim=1536, hidden=2048, heads=12, hd=128, seq=64, nlayers=2, vocab=512), KvDtype.F32, 0, 1e-4),
]


@pytest.mark.parametrize("shape,kvdt,act,tol", LEAN_SHAPES)
def test_short_phase_kernel_matches_oracle(shape, kvdt, act, tol):
    cfg = Config.make(**shape)
    w, orc, dev = pair(cfg, std=0.06, wdt=WeightDtype.BF16, kvdt=kvdt, act=act)
    assert dev.step_kernel() == 2
    ids = synth.make_prompt(5, cfg.vocab, 21)
    lg_o, _, _ = orc.forward_window(ids)
    dev.prefill(ids, want_logits=False)
    tok = int(O.argmax_lower(lg_o[0]))
    for step in range(8):
        a = orc.decode_logits_from_id(tok)
        b = dev.decode_logits_from_id(tok)
        assert rel_err(b, a) < tol, (step, rel_err(b, a))
        tok = int(np.argsort(-a, kind="stable")[step % 3])
    # greedy ids, chained on the device, against the oracle's own greedy loop from here
    n0 = dev.len()
    first = tok
    want, t = [], first
    for _ in range(6):
        lg = orc.decode_logits_from_id(t)
        t = int(O.argmax_lower(lg))
        want.append(t)
    got = dev.decode_greedy_run(first, 6)
    assert dev.len() == n0 + 6
    if kvdt == KvDtype.F32:
        assert [int(x) for x in got] == want
    # per-block top-k candidates and block statistics of the next step (head variants behind the same kernel)
    a = orc.decode_logits_from_id(want[-1] if kvdt == KvDtype.F32 else int(got[-1]))
    if kvdt == KvDtype.F32:
        vals, idxs = dev.decode_token_topk_from_id(want[-1], 4)
        mv, mi = O.merge_topk(vals, idxs, 4)
        assert [int(i) for i in mi] == [int(i) for i in np.argsort(-a, kind="stable")[:4]]


def test_short_phase_kernel_and_general_kernel_agree_and_repeat_bit_for_bit(monkeypatch):
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=96, nlayers=3, vocab=320)
    w = synth.make_weights(cfg, seed=3, std=0.06, round_bf16=True)
    ids = synth.make_prompt(9, cfg.vocab, 17)

    def run():
        dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=KvDtype.F32)
        kind = dev.step_kernel()
        lg = dev.prefill(ids)
        out = [dev.decode_logits_from_id(int(t)) for t in (3, 7, 11, 200)]
        return kind, out
    k1, a = run()
    k2, b = run()
    monkeypatch.setenv("HIPDEC_NO_LEAN", "1")
    k3, c = run()
    assert (k1, k2, k3) == (2, 2, 1)
    for x, y, z in zip(a, b, c):
        assert np.array_equal(x, y)                     # a step is bit-reproducible, whatever ran before it
        assert rel_err(x, z) < 2e-5                     # the two kernels differ in summation order only
