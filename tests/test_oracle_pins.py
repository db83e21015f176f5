"""Pins the CPU oracle before anything is compared against it: the reference's own known answers,
closed forms, invariants and fp64 brute force, chosen so that a dropped term, a wrong index or a
transposed operand fails at least one of them.  Runs on the CPU."""
import ctypes as C
import math

import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import synth
from rustane_amd.hipdec import Config

L = O.lib()


def tiny_cfg(vocab=320, heads=2, kv_heads=None, hd=128, nlayers=2):
    return Config.make(dim=heads * hd, hidden=640, heads=heads, hd=hd, seq=64, nlayers=nlayers, vocab=vocab,
                       kv_heads=kv_heads)


# ------------------------------------------------------------------ reference known answers
def test_rmsnorm_reference_known_answers():
    # crates/engine/src/cpu/rmsnorm.rs:245-277
    x = O.f32([3.0, 4.0]); g = O.f32([1.0, 1.0]); out = np.zeros(2, np.float32)
    L.orc_rmsnorm(O.P(x), O.P(g), O.P(out), 2)
    rms = math.sqrt(12.5 + 1e-5)
    assert abs(out[0] - 3.0 / rms) < 1e-5 and abs(out[1] - 4.0 / rms) < 1e-5
    x = O.f32([1, 2, 3, 4]); g = O.f32([0.5] * 4); out = np.zeros(4, np.float32)
    L.orc_rmsnorm(O.P(x), O.P(g), O.P(out), 4)
    inv = 1.0 / math.sqrt(7.5 + 1e-5)
    np.testing.assert_allclose(out, x * inv * 0.5, atol=1e-5)


def test_rmsnorm_channel_first_equals_per_position():
    # crates/engine/src/cpu/rmsnorm.rs:321-369
    rng = np.random.default_rng(0)
    dim, seq = 24, 7
    x = rng.standard_normal((dim, seq)).astype(np.float32)
    g = rng.standard_normal(dim).astype(np.float32)
    out = np.zeros_like(x); inv = np.zeros(seq, np.float32)
    L.orc_rmsnorm_channel_first(O.P(x), O.P(g), O.P(out), O.P(inv), dim, seq)
    for s in range(seq):
        col = np.ascontiguousarray(x[:, s]); o = np.zeros(dim, np.float32)
        L.orc_rmsnorm(O.P(col), O.P(g), O.P(o), dim)
        np.testing.assert_allclose(out[:, s], o, rtol=1e-6, atol=1e-7)
        ref = col.astype(np.float64) / np.sqrt((col.astype(np.float64) ** 2).mean() + 1e-5) * g
        np.testing.assert_allclose(o, ref, rtol=1e-5, atol=1e-6)


def test_embedding_reference_known_answer():
    # crates/engine/src/cpu/embedding.rs:51-62
    table = O.f32([1, 2, 3, 4, 5, 6]); ids = np.array([2, 0, 1], np.uint32); out = np.zeros(6, np.float32)
    L.orc_embedding(O.P(table), 2, O.PU(ids), 3, O.P(out))
    assert out.tolist() == [5.0, 6.0, 1.0, 2.0, 3.0, 4.0]


# ------------------------------------------------------------------ RoPE
def test_rope_closed_form_and_invariants():
    hd, heads = 64, 3
    rng = np.random.default_rng(1)
    x0 = rng.standard_normal(heads * hd).astype(np.float32)
    x = x0.copy(); L.orc_rope_inplace(O.P(x), heads, hd, 0)
    np.testing.assert_array_equal(x, x0)                       # position 0 is the identity
    for pos in (1, 17, 500):
        x = x0.copy(); L.orc_rope_inplace(O.P(x), heads, hd, pos)
        xe = x0.reshape(heads, hd // 2, 2).astype(np.float64)
        i = np.arange(hd // 2)
        theta = pos / 10000.0 ** (2.0 * i / hd)                # sdpa_fwd.rs:23, lib.rs:1401
        ref = np.empty_like(xe)
        ref[..., 0] = xe[..., 0] * np.cos(theta) - xe[..., 1] * np.sin(theta)
        ref[..., 1] = xe[..., 1] * np.cos(theta) + xe[..., 0] * np.sin(theta)
        np.testing.assert_allclose(x.reshape(heads, hd // 2, 2), ref, atol=2e-4)
        pn = (x.reshape(-1, 2).astype(np.float64) ** 2).sum(1)
        np.testing.assert_allclose(pn, (x0.reshape(-1, 2).astype(np.float64) ** 2).sum(1), rtol=1e-5)
    # <rope(q,m), rope(k,n)> depends on m - n only
    q0 = rng.standard_normal(hd).astype(np.float32); k0 = rng.standard_normal(hd).astype(np.float32)

    def dot(m, n):
        q = q0.copy(); k = k0.copy()
        L.orc_rope_inplace(O.P(q), 1, hd, m); L.orc_rope_inplace(O.P(k), 1, hd, n)
        return float(q.astype(np.float64) @ k.astype(np.float64))
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-3
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-3                   # and it is not symmetric


def test_rope_table_matches_inplace():
    seq, hd = 40, 128
    ct = np.zeros((seq, hd // 2), np.float32); st = np.zeros_like(ct)
    L.orc_rope_table(seq, hd, O.P(ct), O.P(st))
    x0 = np.arange(hd, dtype=np.float32) / 10
    x = x0.copy(); L.orc_rope_inplace(O.P(x), 1, hd, 33)
    e, o = x0[0::2], x0[1::2]
    np.testing.assert_array_equal(x[0::2], e * ct[33] - o * st[33])
    np.testing.assert_array_equal(x[1::2], o * ct[33] + e * st[33])


# ------------------------------------------------------------------ matrix products
def test_gemm_index_conventions_against_fp64_loops():
    rng = np.random.default_rng(2)
    T, D, Oc = 5, 13, 9
    X = rng.standard_normal((T, D)).astype(np.float32)
    W = rng.standard_normal(D * Oc).astype(np.float32)
    Y = np.zeros((T, Oc), np.float32)
    L.orc_gemm_in_major(O.P(X), T, D, O.P(W), Oc, O.P(Y))
    ref = np.zeros((T, Oc))
    for t in range(T):                    # tests/phase4_pretraining_checks.rs:750-763: w1[d*hidden + h]
        for o in range(Oc):
            ref[t, o] = sum(float(X[t, d]) * float(W[d * Oc + o]) for d in range(D))
    np.testing.assert_allclose(Y, ref, rtol=1e-5, atol=1e-5)
    Y2 = np.zeros((T, Oc), np.float32)
    W2 = rng.standard_normal(Oc * D).astype(np.float32)
    L.orc_gemm_out_major(O.P(X), T, D, O.P(W2), Oc, O.P(Y2))
    for t in range(T):                    # :774-784: w2[d*hidden + h] with d the output
        for o in range(Oc):
            ref[t, o] = sum(float(X[t, k]) * float(W2[o * D + k]) for k in range(D))
    np.testing.assert_allclose(Y2, ref, rtol=1e-5, atol=1e-5)
    # large, ragged tile shapes against numpy fp64
    T, D, Oc = 19, 70, 1031
    X = rng.standard_normal((T, D)).astype(np.float32); W = rng.standard_normal((D, Oc)).astype(np.float32)
    Y = np.zeros((T, Oc), np.float32)
    L.orc_gemm_in_major(O.P(X), T, D, O.P(W), Oc, O.P(Y))
    np.testing.assert_allclose(Y, X.astype(np.float64) @ W.astype(np.float64), rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ attention
def _attend(cfg, q, kc, vc, n):
    oc = O.OrcConfig(cfg.dim, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.hd, cfg.seq, cfg.nlayers, cfg.vocab,
                     cfg.q_dim, cfg.kv_dim, cfg.gqa_ratio, 0)
    out = np.zeros(cfg.q_dim, np.float32); sc = np.zeros(cfg.seq, np.float32)
    L.orc_attend_row(C.byref(oc), O.P(O.f32(q)), O.P(O.f32(kc)), O.P(O.f32(vc)), n, O.P(out), O.P(sc))
    return out


@pytest.mark.parametrize("heads,kv_heads", [(2, 2), (4, 2)])
def test_attention_brute_force_and_special_cases(heads, kv_heads):
    cfg = tiny_cfg(heads=heads, kv_heads=kv_heads, hd=64)
    rng = np.random.default_rng(3)
    n = 11
    q = rng.standard_normal(cfg.q_dim).astype(np.float32)
    kc = rng.standard_normal((cfg.seq, cfg.kv_dim)).astype(np.float32)
    vc = rng.standard_normal((cfg.seq, cfg.kv_dim)).astype(np.float32)
    out = _attend(cfg, q, kc, vc, n)
    for h in range(heads):
        g = h // (heads // kv_heads)                       # lib.rs:1438 kvh = qh / GQA_RATIO
        qh = q[h * 64:(h + 1) * 64].astype(np.float64)
        K = kc[:n, g * 64:(g + 1) * 64].astype(np.float64); Vv = vc[:n, g * 64:(g + 1) * 64].astype(np.float64)
        s = K @ qh / math.sqrt(64)
        p = np.exp(s - s.max()); p /= p.sum()
        np.testing.assert_allclose(out[h * 64:(h + 1) * 64], p @ Vv, rtol=1e-4, atol=1e-5)
    # n = 1 returns v0 whatever q is
    out1 = _attend(cfg, q, kc, vc, 1)
    for h in range(heads):
        g = h // (heads // kv_heads)
        np.testing.assert_allclose(out1[h * 64:(h + 1) * 64], vc[0, g * 64:(g + 1) * 64], rtol=1e-6)
    # identical keys give the mean of the values
    kc2 = np.tile(kc[:1], (cfg.seq, 1))
    outm = _attend(cfg, q, kc2, vc, n)
    for h in range(heads):
        g = h // (heads // kv_heads)
        np.testing.assert_allclose(outm[h * 64:(h + 1) * 64], vc[:n, g * 64:(g + 1) * 64].mean(0), rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------------ whole model
def numpy_forward(cfg, w, ids, act=0):
    """An independent fp64 statement of the full-window forward, written with matrix products
    from the formulas (embedding, RMSNorm, RoPE on interleaved pairs, causal softmax, SwiGLU,
    alpha = 1/sqrt(2L), tied head)."""
    D, Q, KV, H, V, hd = cfg.dim, cfg.q_dim, cfg.kv_dim, cfg.hidden, cfg.vocab, cfg.hd
    E = w["embed"].reshape(V, D).astype(np.float64)
    x = E[np.asarray(ids)]
    T = len(ids)
    alpha = 1.0 / math.sqrt(2.0 * cfg.nlayers)

    def rms(v, g):
        return v / np.sqrt((v ** 2).mean(-1, keepdims=True) + 1e-5) * g.astype(np.float64)

    def rope(m, nh):
        m = m.reshape(T, nh, hd // 2, 2)
        theta = np.arange(T)[:, None] / 10000.0 ** (2.0 * np.arange(hd // 2)[None, :] / hd)
        c, s = np.cos(theta)[:, None, :], np.sin(theta)[:, None, :]
        out = np.stack([m[..., 0] * c - m[..., 1] * s, m[..., 1] * c + m[..., 0] * s], -1)
        return out.reshape(T, nh * hd)
    for lw in w["layers"]:
        xn = rms(x, lw["gamma1"])
        q = rope(xn @ lw["wq"].reshape(D, Q).astype(np.float64), cfg.heads)
        k = rope(xn @ lw["wk"].reshape(D, KV).astype(np.float64), cfg.kv_heads)
        v = xn @ lw["wv"].reshape(D, KV).astype(np.float64)
        att = np.zeros((T, Q))
        for h in range(cfg.heads):
            g = h // cfg.gqa_ratio
            s = q[:, h * hd:(h + 1) * hd] @ k[:, g * hd:(g + 1) * hd].T / math.sqrt(hd)
            s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
            p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
            att[:, h * hd:(h + 1) * hd] = p @ v[:, g * hd:(g + 1) * hd]
        x2 = x + alpha * (att @ lw["wo"].reshape(Q, D).astype(np.float64))
        xn2 = rms(x2, lw["gamma2"])
        h1 = xn2 @ lw["w1"].reshape(D, H).astype(np.float64)
        h3 = xn2 @ lw["w3"].reshape(D, H).astype(np.float64)
        if act == 1:
            lr = np.where(h1 > 0, h1, 0.5 * h1); gate = lr * lr * h3
        else:
            gate = h1 / (1.0 + np.exp(-h1)) * h3
        x = x2 + alpha * (gate @ lw["w2"].reshape(D, H).astype(np.float64).T)
    xf = rms(x, w["gamma_final"])
    return xf @ E.T


@pytest.mark.parametrize("heads,kv_heads,act", [(2, 2, 0), (4, 2, 0), (2, 2, 1)])
def test_window_forward_matches_independent_fp64_model(heads, kv_heads, act):
    cfg = tiny_cfg(vocab=320, heads=heads, kv_heads=kv_heads, hd=64)
    w = synth.make_weights(cfg, seed=4, std=0.08)
    rng = np.random.default_rng(5)
    for lw in w["layers"]:
        lw["gamma1"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
        lw["gamma2"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
    w["gamma_final"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    orc = O.Oracle(cfg, w, ffn_activation=act)
    lg, _, _ = orc.forward_window(np.array(ids, np.uint32), n_logit_rows=len(ids))
    ref = numpy_forward(cfg, w, ids, act)
    assert np.abs(lg - ref).max() / np.abs(ref).max() < 2e-5
    cap = 1.5
    lgc, _, _ = O.Oracle(cfg, w, ffn_activation=act).forward_window(np.array(ids, np.uint32), softcap=cap,
                                                                    n_logit_rows=len(ids))
    np.testing.assert_allclose(lgc, cap * np.tanh(ref / cap), atol=3e-5)


def test_cached_step_equals_window_row_and_greedy_ids():
    # the property crates/engine/tests/auto_kv_decode.rs:67-134 asserts
    cfg = tiny_cfg(vocab=320)
    w = synth.make_weights(cfg, seed=6, std=0.08)
    ids = np.array([7, 3, 11, 200, 5, 319, 0, 42, 9], np.uint32)
    lg_all, k_cf, v_cf = O.Oracle(cfg, w).forward_window(ids, n_logit_rows=len(ids), want_caches=True)
    orc = O.Oracle(cfg, w)
    for t, tok in enumerate(ids):
        lg = orc.decode_logits_from_id(int(tok))
        assert np.abs(lg - lg_all[t]).max() < 1e-5
        assert O.argmax_lower(lg) == O.argmax_lower(lg_all[t])
    # seeding from the channel-first caches of the window forward gives the same next step
    o2 = O.Oracle(cfg, w)
    o2.set_len(5)
    for l in range(cfg.nlayers):
        o2.seed_layer_cache_from_channel_first(l, 5, k_cf[l], v_cf[l])
    lg5 = o2.decode_logits_from_id(int(ids[5]))
    assert np.abs(lg5 - lg_all[5]).max() < 1e-5
    kc = o2.kcache(0)
    np.testing.assert_array_equal(kc[:5], k_cf[0][:, :5].T)        # lib.rs:228-234 transpose
    assert not kc[6:].any()


def test_zero_wo_w2_collapses_to_head_of_embedding():
    # the reference's own decode tests run in this regime (crates/engine/src/layer.rs:706-709)
    cfg = tiny_cfg(vocab=320)
    w = synth.make_weights(cfg, seed=8, std=0.05)
    for lw in w["layers"]:
        lw["wo"][:] = 0; lw["w2"][:] = 0
    orc = O.Oracle(cfg, w)
    orc.decode_logits_from_id(5)
    lg = orc.decode_logits_from_id(17)
    E = w["embed"].reshape(cfg.vocab, cfg.dim).astype(np.float64)
    e = E[17]
    ref = E @ (e / np.sqrt((e ** 2).mean() + 1e-5))
    np.testing.assert_allclose(lg, ref, rtol=1e-4, atol=1e-5)


def test_naive_and_cached_loops_agree():
    cfg = tiny_cfg(vocab=320)
    w = synth.make_weights(cfg, seed=9, std=0.08)
    prompt = np.array([4, 8, 15], np.uint32)
    for (T, k) in ((0.0, 0), (0.8, 4)):
        oa, ob = O.Oracle(cfg, w), O.Oracle(cfg, w)
        lg, _, _ = oa.forward_window(prompt)
        ob.forward_window(prompt)
        s_naive, g_naive = oa.run_naive_sample(prompt, lg[0], 10, T, k, seed=7)
        s_cached, g_cached = ob.run_cached_sample(prompt, lg[0], 10, T, k, seed=7)
        np.testing.assert_array_equal(s_naive, s_cached)      # one draw per token on both paths
        np.testing.assert_array_equal(g_naive, g_cached)


def test_suffix_equals_fresh_prompt():
    # crates/engine/src/inference.rs:1001-1033
    cfg = tiny_cfg(vocab=320)
    w = synth.make_weights(cfg, seed=10, std=0.08)
    base, suffix = np.array([1, 2, 3], np.uint32), np.array([4, 5], np.uint32)
    full = np.concatenate([base, suffix])
    oa = O.Oracle(cfg, w)
    lg_base, _, _ = oa.forward_window(base)
    # the suffix path: logits of the last suffix token come from the token loop
    lg = None
    for t in suffix:
        lg = oa.decode_logits_from_id(int(t))
    oa.set_len(len(base))
    s1, _ = oa.run_cached_sample(full, lg, 6, 0.8, 4, seed=17, suffix=suffix)
    ob = O.Oracle(cfg, w)
    lg_full, _, _ = ob.forward_window(full)
    s2, _ = ob.run_cached_sample(full, lg_full[0], 6, 0.8, 4, seed=17)
    np.testing.assert_array_equal(s1, s2)


# ------------------------------------------------------------------ heads
def sort_topk(x, k):
    order = sorted(range(len(x)), key=lambda i: (-x[i], i))
    return order[:k]


def test_argmax_rules_on_ties():
    x = O.f32([1.0, 5.0, 5.0, -2.0, 5.0])
    assert O.argmax_lower(x) == 1          # GPU rule: lower index, lib.rs:1553
    assert O.argmax_last(x) == 4           # Iterator::max_by returns the last maximum, inference.rs:778-783
    z = O.f32([0.0, -0.0, 0.0])
    assert O.argmax_last(z) == 2           # total_cmp: -0.0 < +0.0
    assert O.argmax_lower(O.f32([-np.inf, -np.inf])) == 0


@pytest.mark.parametrize("V", [64, 320, 777])
def test_block_topk_and_merge_against_sort(V):
    rng = np.random.default_rng(V)
    x = rng.standard_normal(V).astype(np.float32)
    x[rng.integers(0, V, 20)] = 1.25          # ties
    x[5] = np.inf; x[6] = -np.inf
    for k in (1, 4, 32):
        vals, idxs = O.block_topk(x, k)
        B = (V + 255) // 256
        for b in range(B):
            blk = x[b * 256:(b + 1) * 256]
            want = sort_topk(blk.tolist(), k)
            got = idxs[b * k:(b + 1) * k]
            for r in range(k):
                if r < len(want) and blk[want[r]] > -np.inf:
                    assert got[r] == b * 256 + want[r]
                    assert vals[b * k + r] == blk[want[r]]
                else:
                    assert np.isneginf(vals[b * k + r])
        mv, mi = O.merge_topk(vals, idxs, k)
        # the merge sees only each block's k survivors and skips non-finite values (decode.rs:229),
        # so a +inf logit uses up one slot of its block and is then dropped
        surv = []
        for b in range(B):
            blk = x[b * 256:(b + 1) * 256].tolist()
            surv += [b * 256 + i for i in sort_topk(blk, k) if np.isfinite(blk[i])]
        want = sorted(surv, key=lambda i: (-x[i], i))[:k]
        assert mi.tolist() == want
        assert mv.tolist() == [x[i] for i in want]


def test_block_stats_lse_identity_and_materialise():
    rng = np.random.default_rng(11)
    V = 777
    x = (3 * rng.standard_normal(V)).astype(np.float32)
    for T, cap in ((0.8, 0.0), (1.3, 4.0)):
        mx, sm = O.block_stats(x, 1.0 / T, cap)
        z = (cap * np.tanh(x.astype(np.float64) / cap) if cap > 0 else x.astype(np.float64)) / T
        g = z.max()
        lhs = (np.exp(mx.astype(np.float64) - g) * sm).sum()
        assert abs(lhs - np.exp(z - g).sum()) / lhs < 1e-5
        for b in range(len(mx)):
            assert abs(mx[b] - z[b * 256:(b + 1) * 256].max()) < 1e-5
        blk = O.materialize_block(x, 3, cap)
        assert blk.size == 777 - 768
        np.testing.assert_allclose(blk, (z * T)[768:], atol=1e-5)


# ------------------------------------------------------------------ RNG and samplers
def test_lcg_known_answers():
    # inference.rs:759-768, constants checked with Python integers
    s = 7
    r = O.Rng(7)
    for _ in range(5):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        assert r.next_u64() == s
    s2 = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
    assert r.next_f32() == np.float32(s2 >> 40) / np.float32(1 << 24)
    r0 = O.Rng(0)
    assert r0.next_u64() == 1442695040888963407


def test_samplers_follow_the_softmax_distribution():
    rng = np.random.default_rng(12)
    logits = rng.standard_normal(6).astype(np.float32)
    T = 0.7
    p = np.exp(logits.astype(np.float64) / T); p /= p.sum()
    counts = np.zeros(6)
    r = O.Rng(99)
    N = 20000
    for _ in range(N):
        counts[L.orc_sample_softmax_index(O.P(logits), 6, T, r.ref)] += 1
    assert np.abs(counts / N - p).max() < 0.015
    # top-k restricted sampling only ever returns the k best, in proportion
    counts = np.zeros(6)
    for _ in range(N):
        counts[L.orc_sample_next(O.P(logits), 6, T, 3, r.ref)] += 1
    best = sort_topk(logits.tolist(), 3)
    assert counts[[i for i in range(6) if i not in best]].sum() == 0
    pk = p[best] / p[best].sum()
    assert np.abs(counts[best] / N - pk).max() < 0.015


def test_sampler_inverse_cdf_is_exact_for_a_given_draw():
    logits = O.f32([0.0, math.log(3.0)])      # weights 1/4 and 3/4 at T = 1
    # find seeds whose first uniform falls on either side of 1/4 (index order: walk from index 0)
    for seed in range(40):
        r = O.Rng(seed); u = O.Rng(seed).next_f32()
        got = L.orc_sample_softmax_index(O.P(logits), 2, 1.0, r.ref)
        w0 = math.exp(0.0 - math.log(3.0))
        assert got == (0 if u * (w0 + 1.0) <= w0 + 1e-7 else 1) or abs(u * (w0 + 1.0) - w0) < 1e-5


def test_sampler_degenerate_cases():
    r = O.Rng(1)
    assert L.orc_sample_topk_candidates(None, None, 0, 0.8, r.ref) == 0            # inference.rs:824-826
    idxs = np.array([9, 4], np.uint32); lg = O.f32([1.0, 0.5])
    assert L.orc_sample_topk_candidates(O.PU(idxs), O.P(lg), 2, 0.0, r.ref) == 9   # T <= 0 -> first
    assert L.orc_sample_topk_candidates(O.PU(idxs), O.P(lg), 1, 0.8, r.ref) == 9
    x = O.f32([0.0, 1e30, -1.0])
    assert L.orc_sample_softmax_index(O.P(x), 3, 1e-38, r.ref) == 1                # sum not finite -> argmax
    assert L.orc_sample_next(O.P(x), 3, 0.0, 0, r.ref) == 1                        # greedy
    assert L.orc_sample_next(O.P(x), 3, 0.9, 1, r.ref) == 1                        # top_k == 1 is greedy
    mx = O.f32([-np.inf, -np.inf]); sm = O.f32([0, 0])
    assert L.orc_sample_block_from_stats(O.P(mx), O.P(sm), 2, r.ref) == 0          # inference.rs:861-863


def _block_draw_expected(maxes, sums, u):
    """The block inference.rs:851-891 must choose for the uniform u, in float64 from the definition:
    weights exp(max_b - gmax) * sum_b (0 where max or sum is not finite or sum <= 0), inverse CDF in
    block order.  Returns (block, margin) with margin = relative distance of u * total to the nearest
    cumulative threshold (draws closer than float32 round-off to a threshold are not decidable)."""
    mx, sm = np.asarray(maxes, np.float64), np.asarray(sums, np.float64)
    fin = np.isfinite(mx)
    g = mx[fin].max()
    ok = fin & np.isfinite(sm) & (sm > 0)
    w = np.where(ok, np.exp(np.where(ok, mx, g) - g) * np.where(ok, sm, 0.0), 0.0)
    cum = np.cumsum(w)
    x = float(u) * cum[-1]
    blk = int(np.searchsorted(cum, x, side="left"))
    live = cum[np.concatenate([[True], np.diff(cum) > 0])]
    return min(blk, len(w) - 1), float(np.abs(live - x).min() / cum[-1])


@pytest.mark.parametrize("case", ["plain", "huge_maxes", "tiny_maxes", "dead_blocks", "short_last_block"])
def test_block_draw_from_stats_inverse_cdf_against_float64(case):
    """orc_sample_block_from_stats (inference.rs:851-891) against the float64 definition, for uniforms on
    either side of every threshold.  The cases are chosen so that a dropped `* sum_b`, a dropped
    `- gmax` (overflow / underflow of exp), a block order other than 0..B-1 or a weight for a block
    with non-finite statistics each pick a different block."""
    if case == "plain":
        mx, sm = [1.0, 0.2, 1.5, -0.3, 0.9, 1.4], [40.0, 200.0, 3.0, 120.0, 77.0, 9.0]
    elif case == "huge_maxes":           # exp(max) overflows float32 without the shift by gmax
        mx, sm = [95.0, 99.5, 97.0, 100.0, 98.0], [30.0, 2.0, 50.0, 1.5, 20.0]
    elif case == "tiny_maxes":           # exp(max) underflows to 0 without the shift
        mx, sm = [-200.0, -201.0, -199.5, -203.0], [10.0, 60.0, 5.0, 250.0]
    elif case == "dead_blocks":          # non-finite max / sum and sum <= 0 carry no weight (inference.rs:861-866)
        mx = [0.5, np.inf, 1.0, -np.inf, 0.8, 0.1, np.nan, 0.7, 0.3]
        sm = [12.0, 5.0, np.nan, 9.0, 0.0, 30.0, 4.0, -25.0, 8.0]
    else:                                # a last block of few rows: its sum is what keeps it rare
        mx, sm = [2.0, 2.1, 1.9, 2.05], [180.0, 190.0, 170.0, 3.0]
    mxa, sma = O.f32(mx), O.f32(sm)
    hit = np.zeros(len(mx), int)
    decided = 0
    for seed in range(3000):
        u = O.Rng(seed).next_f32()
        want, margin = _block_draw_expected(mxa, sma, u)
        if margin < 1e-5:
            continue
        r = O.Rng(seed)
        got = L.orc_sample_block_from_stats(O.P(mxa), O.P(sma), len(mx), r.ref)
        assert got == want, (case, seed, u, got, want)
        assert r.s.value == (seed * 6364136223846793005 + 1442695040888963407) % (1 << 64)     # exactly one draw
        hit[got] += 1
        decided += 1
    assert decided > 2900
    mx64, sm64 = np.asarray(mxa, np.float64), np.asarray(sma, np.float64)
    live = np.isfinite(mx64) & np.isfinite(sm64) & (sm64 > 0)
    assert np.all(hit[live] > 0) and np.all(hit[~live] == 0)        # both sides of every threshold were visited


def test_block_then_token_sampling_reproduces_the_softmax_distribution():
    """The two draws of the cached full-vocabulary path (block from the statistics, inference.rs:851-891,
    then the token inside the block, :893-921) must together sample softmax(logits / T): block marginals
    and token probabilities over 40 000 draws at V = 777 (three full blocks and one of 9 rows)."""
    rng = np.random.default_rng(21)
    V, T = 777, 0.8
    logits = (rng.standard_normal(V) * 1.5).astype(np.float32)
    logits[770:] += 2.0                                    # the short block is not negligible
    p = np.exp((logits.astype(np.float64) - logits.max()) / T); p /= p.sum()
    inv_t = float(np.float32(1.0) / np.float32(T))
    mx, sm = O.block_stats(logits, inv_t, 0.0)
    B = len(mx)
    r = O.Rng(2024)
    N = 40000
    counts = np.zeros(V)
    for _ in range(N):
        b = L.orc_sample_block_from_stats(O.P(mx), O.P(sm), B, r.ref)
        blk = O.materialize_block(logits, b, 0.0)
        counts[L.orc_sample_block_logits(b * 256, O.P(blk), blk.size, T, r.ref)] += 1
    pb = np.array([p[b * 256:(b + 1) * 256].sum() for b in range(B)])
    cb = np.array([counts[b * 256:(b + 1) * 256].sum() for b in range(B)])
    assert np.abs(cb / N - pb).max() < 4.0 * np.sqrt(0.25 / N)                 # 4 sigma of a block frequency
    # token level: chi-square of the observed counts against softmax (cells with expectation >= 5)
    e = p * N
    cells = e >= 5.0
    chi2 = float((((counts - e) ** 2) / e)[cells].sum()) + (counts[~cells].sum() - e[~cells].sum()) ** 2 / max(e[~cells].sum(), 1.0)
    dof = int(cells.sum())
    assert chi2 < dof + 5.0 * np.sqrt(2.0 * dof), (chi2, dof)
    assert np.abs(counts / N - p).max() < 0.01


def test_fullvocab_cached_path_draws_twice_per_token():
    # inference.rs:602-617 (block, then token inside the block) against :786-788 (one draw)
    cfg = tiny_cfg(vocab=320)
    w = synth.make_weights(cfg, seed=13, std=0.08)
    prompt = np.array([1, 2, 3], np.uint32)
    orc = O.Oracle(cfg, w)
    lg, _, _ = orc.forward_window(prompt)
    steps = 5
    sampled, _ = orc.run_cached_sample(prompt, lg[0], steps, 1.0, 0, seed=3)
    # replay by hand with the primitive samplers
    o2 = O.Oracle(cfg, w); o2.forward_window(prompt)
    r = O.Rng(3)
    cur = L.orc_sample_next(O.P(O.f32(lg[0])), cfg.vocab, 1.0, 0, r.ref)
    mine = [cur]
    for _ in range(steps - 1):
        raw = o2.decode_logits_from_id(int(cur))
        mx, sm = O.block_stats(raw, 1.0, 0.0)
        b = L.orc_sample_block_from_stats(O.P(mx), O.P(sm), len(mx), r.ref)
        blk = O.materialize_block(raw, b, 0.0)
        cur = L.orc_sample_block_logits(b * 256, O.P(blk), blk.size, 1.0, r.ref)
        mine.append(cur)
    assert sampled.tolist() == mine
    s = 3
    for _ in range(1 + 2 * (steps - 1)):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
    assert r.s.value == s


def test_fill_input_window_slides():
    # inference.rs:751-757
    gen = np.arange(1, 11, dtype=np.uint32)
    out = np.full(4, 99, np.uint32)
    assert L.orc_fill_input_window(O.PU(gen), 10, 4, O.PU(out)) == 4
    assert out.tolist() == [7, 8, 9, 10]
    out = np.full(16, 99, np.uint32)
    assert L.orc_fill_input_window(O.PU(gen), 10, 16, O.PU(out)) == 10
    assert out.tolist() == list(range(1, 11)) + [0] * 6


# ------------------------------------------------------------------ weight formats
def e4m3_table():
    return np.array([L.orc_e4m3_to_f32(b) for b in range(256)], np.float64)


def test_e4m3_decode_table_and_roundtrip():
    t = e4m3_table()
    assert t[0x7e] == 448.0 and t[0x01] == 2.0 ** -9 and t[0x08] == 2.0 ** -6 and t[0x38] == 1.0
    assert np.isnan(t[0x7f]) and np.isnan(t[0xff])
    for b in range(256):
        if not np.isnan(t[b]):
            assert L.orc_f32_to_e4m3(float(t[b])) == (b if t[b] != 0 or b == 0 else b)


def test_e4m3_encode_is_nearest_even():
    t = e4m3_table()
    pos = np.array([b for b in range(0x7f)])                  # non-negative finite codes, ascending values
    vals = t[pos]
    rng = np.random.default_rng(14)
    xs = np.concatenate([rng.uniform(0, 470, 3000), rng.uniform(0, 0.05, 2000), (vals[:-1] + vals[1:]) / 2])
    for x in xs.astype(np.float32):
        code = L.orc_f32_to_e4m3(float(x))
        d = np.abs(vals - float(x))
        best = d.min()
        cands = pos[d == best]
        want = cands[0] if len(cands) == 1 else [c for c in cands if c % 2 == 0][0]   # tie -> even mantissa
        assert code == want, (x, code, want)
        assert L.orc_f32_to_e4m3(float(-x)) == (want | 0x80)


def test_quantisers_properties():
    rng = np.random.default_rng(15)
    O_, K = 6, 256
    W = (0.05 * rng.standard_normal((O_, K))).astype(np.float32)
    W[2] = 0
    dq = np.empty_like(W); sc = np.empty(O_, np.float32); q8 = np.empty((O_, K), np.uint8)
    L.orc_quant_fp8_rows(O.P(W), O_, K, q8.ctypes.data_as(C.POINTER(C.c_uint8)), O.P(sc), O.P(dq))
    np.testing.assert_allclose(sc[[0, 1, 3, 4, 5]], np.abs(W[[0, 1, 3, 4, 5]]).max(1) / 448.0, rtol=1e-6)
    assert sc[2] == 1.0 and not dq[2].any()
    assert np.abs(dq - W).max() <= np.abs(W).max() * 2 ** -4 + 1e-9          # 3 mantissa bits
    for o in (0, 1):
        am = np.abs(W[o]).argmax()
        assert abs(abs(dq[o, am]) - abs(W[o, am])) < 1e-6 * abs(W[o, am]) + 1e-9   # amax maps to 448 exactly
    q4 = np.empty((O_, K), np.int8); sc4 = np.empty((O_, K // 128), np.float32); dq4 = np.empty_like(W)
    L.orc_quant_int4_g128(O.P(W), O_, K, q4.ctypes.data_as(C.POINTER(C.c_int8)), O.P(sc4), O.P(dq4))
    assert q4.min() >= -8 and q4.max() <= 7
    np.testing.assert_array_equal(dq4, q4.astype(np.float32) * np.repeat(sc4, 128, axis=1))
    assert np.abs(dq4 - W).max() <= np.repeat(sc4, 128, axis=1).max() * 0.51
    b = sc4.view(np.uint32)
    assert not (b & 0xffff).any()                                           # scales are bf16 values
