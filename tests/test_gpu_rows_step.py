"""GPU parity of the multi-row step whose layers run as one persistent launch (hipdec_rows.h): bf16
weights, at most 8 rows, dimensions that are multiples of 256.  Every row is checked against its own
CPU oracle, as in test_gpu_batch_decode.py (the reference draws its samples one after the other,
crates/engine/src/inference.rs:247-262, :561), and against the same step run as one kernel per product."""
import os

import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import synth
from rustane_amd.hipdec import Config, HipDecodeModel, KvDtype, WeightDtype

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / max(np.abs(b).max(), 1e-30))


def setup(cfg, rows, n_prompt, kvdt=KvDtype.F32, std=0.07, seed=17, act=0):
    w = synth.make_weights(cfg, seed=seed, std=std, round_bf16=True)
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=kvdt, ffn_activation=act)
    ids = synth.make_prompt(3, cfg.vocab, n_prompt)
    dev.prefill(ids, want_logits=False)
    orcs = []
    for _ in range(rows):
        o = O.Oracle(cfg, w, kv_round_bf16=(kvdt == KvDtype.BF16), ffn_activation=act)
        o.forward_window(ids)
        orcs.append(o)
    return w, dev, orcs, ids


def walk(dev, orcs, cfg, rows, steps, tol):
    toks = np.array([(7 * r + 1) % cfg.vocab for r in range(rows)], np.uint32)
    for step in range(steps):
        got = dev.decode_logits_from_ids_batch(toks)
        want = np.stack([orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)])
        for r in range(rows):
            assert rel_err(got[r], want[r]) < tol, (step, r, rel_err(got[r], want[r]))
        toks = np.array([np.argsort(-want[r], kind="stable")[r % 4] for r in range(rows)], np.uint32)


@pytest.mark.parametrize("rows,n_prompt", [(1, 9), (3, 20), (8, 40)])
def test_rows_kernel_matches_sequential_oracles(rows, n_prompt):
    cfg = Config.make(dim=256, hidden=512, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w, dev, orcs, ids = setup(cfg, rows, n_prompt)
    dev.batch_begin(rows)
    assert dev.batch_layers_in_one_launch()
    walk(dev, orcs, cfg, rows, 6, 1e-4)
    dev.batch_end()
    assert dev.len() == n_prompt
    fresh = O.Oracle(cfg, w)
    fresh.forward_window(ids)
    assert rel_err(dev.decode_logits_from_id(5), fresh.decode_logits_from_id(5)) < 1e-4


def test_rows_kernel_bf16_cache_gqa_hd64_leaky_relu_odd_layers():
    cfg = Config.make(dim=512, hidden=768, heads=8, hd=64, seq=96, nlayers=3, vocab=600, kv_heads=4)
    rows = 5
    w, dev, orcs, ids = setup(cfg, rows, 33, kvdt=KvDtype.BF16, std=0.05, act=1)
    dev.batch_begin(rows)
    assert dev.batch_layers_in_one_launch()
    walk(dev, orcs, cfg, rows, 7, 2e-3)
    dev.batch_end()


def test_rows_kernel_split_count_grows_and_batches_reopen():
    # fp32 cache, head dimension 128: a split covers 64 cache rows, so the split count goes 1 -> 2 when the
    # 65th position is attended (an odd layer count makes consecutive launches start with different stamps);
    # then the same model opens batches of other row counts, each from cleared exchange buffers
    cfg = Config.make(dim=256, hidden=512, heads=2, hd=128, seq=128, nlayers=3, vocab=320)
    rows = 3
    w, dev, orcs, ids = setup(cfg, rows, 60)
    dev.batch_begin(rows)
    assert dev.batch_layers_in_one_launch()
    walk(dev, orcs, cfg, rows, 9, 1e-4)
    dev.batch_end()
    for rows2 in (8, 2):
        orcs2 = []
        for _ in range(rows2):
            o = O.Oracle(cfg, w)
            o.forward_window(ids)
            orcs2.append(o)
        dev.batch_begin(rows2)
        assert dev.batch_layers_in_one_launch()
        walk(dev, orcs2, cfg, rows2, 3, 1e-4)
        dev.batch_end()


@pytest.mark.parametrize("kvdt,tol", [(KvDtype.F32, 2e-5), (KvDtype.BF16, 5e-4)])
def test_rows_kernel_equals_one_kernel_per_product(kvdt, tol):
    # (with a bf16 cache a last-bit difference in a key or value moves its rounding: looser)
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=96, nlayers=2, vocab=512)
    rows = 8
    w = synth.make_weights(cfg, seed=5, std=0.06, round_bf16=True)
    ids = synth.make_prompt(3, cfg.vocab, 40)
    outs = {}
    for off in ("0", "1"):
        os.environ["HIPDEC_NO_ROWS_KERNEL"] = off
        try:
            dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=kvdt)
            dev.prefill(ids, want_logits=False)
            dev.batch_begin(rows)
            assert dev.batch_layers_in_one_launch() == (off == "0")
            toks = np.arange(1, rows + 1, dtype=np.uint32)
            seq = []
            for _ in range(5):
                lg = dev.decode_logits_from_ids_batch(toks)
                seq.append(lg)
                toks = lg.argmax(axis=1).astype(np.uint32)
            dev.batch_end()
            outs[off] = np.stack(seq)
        finally:
            os.environ.pop("HIPDEC_NO_ROWS_KERNEL", None)
    assert rel_err(outs["0"], outs["1"]) < tol


def test_rows_kernel_not_taken_where_it_does_not_fit():
    # hidden not a multiple of 256; more than 8 rows; 8-bit weights
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=48, nlayers=1, vocab=64)
    w = synth.make_weights(cfg, seed=1, std=0.05, round_bf16=True)
    dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16)
    dev.prefill(synth.make_prompt(3, cfg.vocab, 9), want_logits=False)
    dev.batch_begin(2)
    assert not dev.batch_layers_in_one_launch()
    dev.batch_end()
    cfg = Config.make(dim=256, hidden=512, heads=2, hd=128, seq=48, nlayers=1, vocab=64)
    w = synth.make_weights(cfg, seed=1, std=0.05, round_bf16=True)
    for wdt, rows, want in ((WeightDtype.BF16, 9, False), (WeightDtype.FP8_E4M3, 4, False), (WeightDtype.BF16, 8, True)):
        dev = HipDecodeModel(cfg, w, weight_dtype=wdt)
        dev.prefill(synth.make_prompt(3, cfg.vocab, 9), want_logits=False)
        dev.batch_begin(rows)
        assert dev.batch_layers_in_one_launch() == want
        dev.batch_end()


@pytest.mark.parametrize("T,k,softcap", [(0.0, 0, 0.0), (0.8, 8, 0.0), (1.0, 0, 2.5), (0.9, 40, 3.0)])
def test_session_samples_through_the_rows_kernel_equal_the_oracle_loop(T, k, softcap):
    # The session layer steps the samples of a request together (the reference draws them one after the
    # other, inference.rs:247-262); on a model the one-launch layers take, every sample's stream, greedy or
    # drawn on the device, must equal the oracle's cached loop (inference.rs:542-648).
    from rustane_amd import engine as E
    cfg = Config.make(dim=256, hidden=512, heads=2, hd=128, seq=64, nlayers=3, vocab=1000)
    prompt = [5, 6, 7, 8, 9, 10, 11, 12, 13]
    w = synth.make_weights(cfg, seed=31, std=0.08, round_bf16=True)
    req = E.GenerationRequest(E.DecodeBackendRequest.HIP, steps=10, temperature=T, top_k=k, samples=5, seed=21)
    got = E.InferenceSession(cfg, w, prompt, softcap=softcap, weight_dtype=1).generate(req)
    assert len(got.results) == 5
    full = np.array(prompt, np.uint32)
    for i, r in enumerate(got.results):
        orc = O.Oracle(cfg, w)
        lg, _, _ = orc.forward_window(full, softcap=softcap)
        sampled, gen = orc.run_cached_sample(full, lg[0], req.steps, req.temperature, req.top_k, seed=req.seed + i,
                                             softcap=softcap)
        np.testing.assert_array_equal(r.sampled, sampled)
        np.testing.assert_array_equal(r.generated, gen)


@pytest.mark.parametrize("kvdt", [KvDtype.F32, KvDtype.BF16])
def test_rows_kernel_runs_repeat_bit_for_bit(kvdt):
    # Tolerance 0.0, the reference's style for schedule changes (its auto_*.rs tests): every value this step
    # exchanges is read by value and stamp, in a fixed order, so two runs from fresh models must give the same
    # bits whatever the timing of the workgroups (an odd layer count makes consecutive launches start from
    # different stamps)
    cfg = Config.make(dim=512, hidden=1024, heads=4, hd=128, seq=128, nlayers=3, vocab=1024)
    w = synth.make_weights(cfg, seed=9, std=0.06, round_bf16=True)
    ids = synth.make_prompt(3, cfg.vocab, 40)

    def run():
        dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=kvdt)
        dev.prefill(ids, want_logits=False)
        dev.batch_begin(8)
        assert dev.batch_layers_in_one_launch()
        toks = np.arange(1, 9, dtype=np.uint32)
        out = []
        for _ in range(40):
            lg = dev.decode_logits_from_ids_batch(toks)
            out.append(lg.copy())
            toks = lg.argmax(axis=1).astype(np.uint32)
        dev.batch_end()
        return np.stack(out)

    a, b = run(), run()
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
    assert len(np.unique(a.argmax(axis=2))) > 20          # (the streams are not a fixed point)


@pytest.mark.parametrize("kvdt,tol", [(KvDtype.F32, 2e-4), (KvDtype.BF16, 5e-3)])
def test_rows_kernel_at_the_600m_shape_equals_one_kernel_per_product(kvdt, tol):
    # the workload's own shape (bands of 18 / 32 / 6 weight rows, two tiles in the even phases, six and
    # sixteen steps per wave, 12 heads x 8 rows of attention items in two splits): the same tokens through
    # both forms of the step.  (With a bf16 cache a last-bit difference upstream moves the rounding of a
    # cached value, a 2^-8 step: 1e-3 of the largest logit was measured over 24 layers, the bound for bf16 is
    # 2e-2.)
    cfg = synth.config_600m()
    w = synth.make_weights(cfg, seed=3, std=0.05, round_bf16=True)
    ids = synth.make_prompt(7, cfg.vocab, 300)
    devs = {}
    for off in ("0", "1"):
        os.environ["HIPDEC_NO_ROWS_KERNEL"] = off
        try:
            dev = HipDecodeModel(cfg, w, weight_dtype=WeightDtype.BF16, kv_dtype=kvdt)
            dev.prefill(ids, want_logits=False)
            dev.batch_begin(8)
            assert dev.batch_layers_in_one_launch() == (off == "0")
            devs[off] = dev
        finally:
            os.environ.pop("HIPDEC_NO_ROWS_KERNEL", None)
    toks = np.arange(1, 9, dtype=np.uint32)
    seen = set()
    for step in range(24):
        a = devs["0"].decode_logits_from_ids_batch(toks)
        b = devs["1"].decode_logits_from_ids_batch(toks)
        for r in range(8):
            assert rel_err(a[r], b[r]) < tol, (step, r, rel_err(a[r], b[r]))
        toks = a.argmax(axis=1).astype(np.uint32)
        seen.update(int(t) for t in toks)
    assert len(seen) > 20


def test_rows_kernel_step_profile_is_a_step_like_any_other():
    # hipdec_debug_batch_step_profile runs the build with time stamps: the rows advance by one token exactly as
    # with the plain build, and workgroup 0's stamps come back in order, 16 per layer
    cfg = Config.make(dim=256, hidden=512, heads=2, hd=128, seq=96, nlayers=3, vocab=320)
    rows = 4
    w, dev, orcs, ids = setup(cfg, rows, 20)
    dev.batch_begin(rows)
    toks = np.array([3, 50, 101, 299], np.uint32)
    pr = dev.debug_batch_step_profile(toks).astype(np.int64)
    assert pr.shape == (cfg.nlayers + 1, 16) and dev.batch_steps() == 1
    for l in range(cfg.nlayers):
        assert np.all(pr[l] > 0) and np.all(np.diff(pr[l]) >= 0) and pr[l + 1][0] >= pr[l][15]
    nxt = []
    for r in range(rows):
        nxt.append(O.argmax_lower(orcs[r].decode_logits_from_id(int(toks[r]))))
    toks = np.array(nxt, np.uint32)
    got = dev.decode_logits_from_ids_batch(toks)
    for r in range(rows):
        assert rel_err(got[r], orcs[r].decode_logits_from_id(int(toks[r]))) < 1e-4
    dev.batch_end()
    with pytest.raises(Exception):
        dev.debug_batch_step_profile(toks)                    # no batch open


def test_rows_kernel_wait_that_gives_up_reopens_on_the_kernel_per_product_step():
    """The multi-row layer kernel bounds its waits like the single-row one: with the bound at zero polls (test
    hook, every kernel exits normally) a step reports HIPDEC_ERR_HIP; the reopened batch runs one kernel per
    product and its rows still equal their oracles."""
    from rustane_amd import hipdec
    from rustane_amd.hipdec import HipDecodeError, ERR_HIP
    cfg = Config.make(dim=256, hidden=512, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    rows = 3
    w, dev, orcs, ids = setup(cfg, rows, 20)
    dev.batch_begin(rows)
    assert dev.batch_layers_in_one_launch()
    toks = np.array([1, 8, 15], np.uint32)
    failed = False
    hipdec.set_spin_limit(0, 0)
    try:
        for _ in range(6):
            try:
                got = dev.decode_logits_from_ids_batch(toks)
            except HipDecodeError as e:
                assert e.status == ERR_HIP
                failed = True
                break
            want = np.stack([orcs[r].decode_logits_from_id(int(toks[r])) for r in range(rows)])
            for r in range(rows):
                assert rel_err(got[r], want[r]) < 1e-4
    finally:
        hipdec.set_spin_limit()
    assert failed, "no wait gave up with a zero poll limit"
    dev.batch_end()
    # the oracles of the rows restart from the prompt, like the reopened batch
    orcs = []
    for _ in range(rows):
        o = O.Oracle(cfg, w)
        o.forward_window(ids)
        orcs.append(o)
    dev.batch_begin(rows)
    assert not dev.batch_layers_in_one_launch()
    walk(dev, orcs, cfg, rows, 4, 1e-4)
    dev.batch_end()
