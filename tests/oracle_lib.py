"""ctypes view of oracle/liboracle.so (the CPU checker).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "liboracle.so")

fp = C.POINTER(C.c_float)
u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)


class OrcConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("dim", "hidden", "heads", "kv_heads", "hd", "seq", "nlayers", "vocab",
                                         "q_dim", "kv_dim", "gqa_ratio", "ffn_activation")]


class OrcLayer(C.Structure):
    _fields_ = [(n, fp) for n in ("wq", "wk", "wv", "wo", "w1", "w3", "w2", "gamma1", "gamma2")]


_lib = None


def build_oracle():
    subprocess.run(["make", "-C", ORACLE_DIR, "liboracle.so"], check=True, stdout=subprocess.PIPE,
                   stderr=subprocess.STDOUT)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build_oracle()
        L = C.CDLL(ORACLE_SO)
        L.orc_create.restype = C.c_void_p
        L.orc_create.argtypes = [C.POINTER(OrcConfig), C.POINTER(OrcLayer), fp, fp, C.c_int]
        L.orc_destroy.argtypes = [C.c_void_p]
        L.orc_len.argtypes = [C.c_void_p]
        L.orc_set_len.argtypes = [C.c_void_p, C.c_int]
        L.orc_seed_layer_cache_from_channel_first.argtypes = [C.c_void_p, C.c_int, C.c_int, fp, fp]
        L.orc_kcache.restype = fp
        L.orc_kcache.argtypes = [C.c_void_p, C.c_int]
        L.orc_vcache.restype = fp
        L.orc_vcache.argtypes = [C.c_void_p, C.c_int]
        L.orc_forward_window.argtypes = [C.c_void_p, u32p, C.c_int, C.c_float, C.c_int, fp, fp, fp]
        L.orc_decode_token_from_id.argtypes = [C.c_void_p, C.c_uint32, fp]
        L.orc_decode_token.argtypes = [C.c_void_p, fp, fp]
        L.orc_decode_logits_from_id.argtypes = [C.c_void_p, C.c_uint32, C.c_float, fp]
        L.orc_rmsnorm.argtypes = [fp, fp, fp, C.c_int]
        L.orc_rmsnorm_channel_first.argtypes = [fp, fp, fp, fp, C.c_int, C.c_int]
        L.orc_embedding.argtypes = [fp, C.c_int, u32p, C.c_int, fp]
        L.orc_rope_inplace.argtypes = [fp, C.c_int, C.c_int, C.c_int]
        L.orc_rope_table.argtypes = [C.c_int, C.c_int, fp, fp]
        L.orc_gemm_in_major.argtypes = [fp, C.c_int, C.c_int, fp, C.c_int, fp]
        L.orc_gemm_out_major.argtypes = [fp, C.c_int, C.c_int, fp, C.c_int, fp]
        L.orc_attend_row.argtypes = [C.POINTER(OrcConfig), fp, fp, fp, C.c_int, fp, fp]
        L.orc_argmax_lower.restype = C.c_uint32
        L.orc_argmax_lower.argtypes = [fp, C.c_int]
        L.orc_argmax_last.restype = C.c_uint32
        L.orc_argmax_last.argtypes = [fp, C.c_int]
        L.orc_block_topk.argtypes = [fp, C.c_int, C.c_int, fp, u32p]
        L.orc_merge_topk.argtypes = [fp, u32p, C.c_int, C.c_int, fp, u32p]
        L.orc_topk_candidates.argtypes = [fp, C.c_int, C.c_int, C.c_float, u32p, fp]
        L.orc_block_stats.argtypes = [fp, C.c_int, C.c_float, C.c_float, fp, fp]
        L.orc_materialize_block.argtypes = [fp, C.c_int, C.c_int, C.c_float, fp]
        L.orc_next_u64.restype = C.c_uint64
        L.orc_next_u64.argtypes = [u64p]
        L.orc_next_f32.restype = C.c_float
        L.orc_next_f32.argtypes = [u64p]
        L.orc_sample_softmax_index.restype = C.c_size_t
        L.orc_sample_softmax_index.argtypes = [fp, C.c_int, C.c_float, u64p]
        L.orc_sample_next.restype = C.c_uint32
        L.orc_sample_next.argtypes = [fp, C.c_int, C.c_float, C.c_int, u64p]
        L.orc_sample_topk_candidates.restype = C.c_uint32
        L.orc_sample_topk_candidates.argtypes = [u32p, fp, C.c_int, C.c_float, u64p]
        L.orc_sample_block_from_stats.restype = C.c_size_t
        L.orc_sample_block_from_stats.argtypes = [fp, fp, C.c_int, u64p]
        L.orc_sample_block_logits.restype = C.c_uint32
        L.orc_sample_block_logits.argtypes = [C.c_uint32, fp, C.c_int, C.c_float, u64p]
        L.orc_fill_input_window.argtypes = [u32p, C.c_int, C.c_int, u32p]
        L.orc_run_naive_sample.argtypes = [C.c_void_p, u32p, C.c_int, fp, C.c_float, C.c_int, C.c_float, C.c_int,
                                           C.c_uint64, u32p]
        L.orc_run_cached_sample.argtypes = [C.c_void_p, u32p, C.c_int, fp, u32p, C.c_int, C.c_float, C.c_int,
                                            C.c_float, C.c_int, C.c_uint64, u32p]
        L.orc_f32_to_e4m3.restype = C.c_uint8
        L.orc_f32_to_e4m3.argtypes = [C.c_float]
        L.orc_e4m3_to_f32.restype = C.c_float
        L.orc_e4m3_to_f32.argtypes = [C.c_uint8]
        L.orc_quant_fp8_rows.argtypes = [fp, C.c_int, C.c_int, C.POINTER(C.c_uint8), fp, fp]
        L.orc_quant_int4_g128.argtypes = [fp, C.c_int, C.c_int, C.POINTER(C.c_int8), fp, fp]
        L.orc_transpose.argtypes = [fp, C.c_int, C.c_int, fp]
        L.orc_bf16_round_inplace.argtypes = [fp, C.c_size_t]
        _lib = L
    return _lib


def P(a):
    return a.ctypes.data_as(fp)


def PU(a):
    return a.ctypes.data_as(u32p)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Oracle:
    """The CPU restatement behind one object: window forward, cached steps, heads, samplers."""

    def __init__(self, cfg, weights, kv_round_bf16=False, ffn_activation=0):
        self.L = lib()
        self.cfg = cfg
        oc = OrcConfig(cfg.dim, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.hd, cfg.seq, cfg.nlayers, cfg.vocab,
                       cfg.q_dim, cfg.kv_dim, cfg.gqa_ratio, ffn_activation)
        self._keep = []
        layers = (OrcLayer * cfg.nlayers)()
        for i, lw in enumerate(weights["layers"]):
            for name in ("wq", "wk", "wv", "wo", "w1", "w3", "w2", "gamma1", "gamma2"):
                a = f32(lw[name])
                self._keep.append(a)
                setattr(layers[i], name, P(a))
        self.embed = f32(weights["embed"])
        self.gamma_final = f32(weights["gamma_final"])
        self.h = C.c_void_p(self.L.orc_create(C.byref(oc), layers, P(self.gamma_final), P(self.embed),
                                              int(kv_round_bf16)))

    def close(self):
        if self.h:
            self.L.orc_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def len(self):
        return self.L.orc_len(self.h)

    def set_len(self, n):
        self.L.orc_set_len(self.h, n)

    def forward_window(self, ids, softcap=0.0, n_logit_rows=1, want_caches=False):
        """Runs positions 0..len(ids)-1; returns (logits[n_logit_rows, vocab], k_cf, v_cf)."""
        c = self.cfg
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        logits = np.empty((n_logit_rows, c.vocab), np.float32)
        k_cf = v_cf = None
        if want_caches:
            k_cf = np.zeros((c.nlayers, c.kv_dim, c.seq), np.float32)
            v_cf = np.zeros((c.nlayers, c.kv_dim, c.seq), np.float32)
        rc = self.L.orc_forward_window(self.h, PU(ids), ids.size, softcap, n_logit_rows, P(logits),
                                       P(k_cf) if want_caches else None, P(v_cf) if want_caches else None)
        if rc:
            raise RuntimeError("orc_forward_window rc=%d" % rc)
        return logits, k_cf, v_cf

    def seed_layer_cache_from_channel_first(self, layer, live_len, k_cf, v_cf):
        self.L.orc_seed_layer_cache_from_channel_first(self.h, layer, live_len, P(f32(k_cf)), P(f32(v_cf)))

    def decode_token_from_id(self, tok):
        out = np.empty(self.cfg.dim, np.float32)
        rc = self.L.orc_decode_token_from_id(self.h, tok, P(out))
        if rc:
            raise RuntimeError("orc_decode_token_from_id rc=%d" % rc)
        return out

    def decode_token(self, x_in):
        x = f32(x_in)
        out = np.empty(self.cfg.dim, np.float32)
        rc = self.L.orc_decode_token(self.h, P(x), P(out))
        if rc:
            raise RuntimeError("orc_decode_token rc=%d" % rc)
        return out

    def decode_logits_from_id(self, tok, softcap=0.0):
        out = np.empty(self.cfg.vocab, np.float32)
        rc = self.L.orc_decode_logits_from_id(self.h, tok, softcap, P(out))
        if rc:
            raise RuntimeError("orc_decode_logits_from_id rc=%d" % rc)
        return out

    def kcache(self, layer):
        c = self.cfg
        return np.ctypeslib.as_array(self.L.orc_kcache(self.h, layer), shape=(c.seq, c.kv_dim)).copy()

    def vcache(self, layer):
        c = self.cfg
        return np.ctypeslib.as_array(self.L.orc_vcache(self.h, layer), shape=(c.seq, c.kv_dim)).copy()

    def run_cached_sample(self, prompt_ids, prompt_logits, steps, temperature=0.0, top_k=0, seed=1, softcap=0.0,
                          suffix=()):
        gen = np.zeros(len(prompt_ids) + steps, np.uint32)
        gen[:len(prompt_ids)] = prompt_ids
        sampled = np.zeros(max(steps, 1), np.uint32)
        suf = np.ascontiguousarray(suffix, dtype=np.uint32)
        pl = f32(prompt_logits)
        rc = self.L.orc_run_cached_sample(self.h, PU(gen), len(prompt_ids), P(pl), PU(suf), suf.size, softcap, steps,
                                          temperature, top_k, seed, PU(sampled))
        if rc:
            raise RuntimeError("orc_run_cached_sample rc=%d" % rc)
        return sampled[:steps], gen

    def run_naive_sample(self, prompt_ids, prompt_logits, steps, temperature=0.0, top_k=0, seed=1, softcap=0.0):
        gen = np.zeros(len(prompt_ids) + steps, np.uint32)
        gen[:len(prompt_ids)] = prompt_ids
        sampled = np.zeros(max(steps, 1), np.uint32)
        pl = f32(prompt_logits)
        rc = self.L.orc_run_naive_sample(self.h, PU(gen), len(prompt_ids), P(pl), softcap, steps, temperature, top_k,
                                         seed, PU(sampled))
        if rc:
            raise RuntimeError("orc_run_naive_sample rc=%d" % rc)
        return sampled[:steps], gen


# ---- head / sampler helpers on plain arrays
def argmax_lower(logits):
    a = f32(logits)
    return lib().orc_argmax_lower(P(a), a.size)


def argmax_last(logits):
    a = f32(logits)
    return lib().orc_argmax_last(P(a), a.size)


def block_topk(logits, top_k):
    a = f32(logits)
    B = (a.size + 255) // 256
    vals = np.empty(B * top_k, np.float32)
    idxs = np.empty(B * top_k, np.uint32)
    lib().orc_block_topk(P(a), a.size, top_k, P(vals), PU(idxs))
    return vals, idxs


def merge_topk(vals, idxs, top_k):
    v, i = f32(vals), np.ascontiguousarray(idxs, dtype=np.uint32)
    ov = np.empty(top_k, np.float32)
    oi = np.empty(top_k, np.uint32)
    n = lib().orc_merge_topk(P(v), PU(i), v.size, top_k, P(ov), PU(oi))
    return ov[:n], oi[:n]


def topk_candidates(raw_logits, top_k, softcap=0.0):
    a = f32(raw_logits)
    ov = np.empty(32, np.float32)
    oi = np.empty(32, np.uint32)
    n = lib().orc_topk_candidates(P(a), a.size, top_k, softcap, PU(oi), P(ov))
    return oi[:n], ov[:n]


def block_stats(raw_logits, inv_t, softcap=0.0):
    a = f32(raw_logits)
    B = (a.size + 255) // 256
    mx = np.empty(B, np.float32)
    sm = np.empty(B, np.float32)
    lib().orc_block_stats(P(a), a.size, inv_t, softcap, P(mx), P(sm))
    return mx, sm


def materialize_block(raw_logits, block_idx, softcap=0.0):
    a = f32(raw_logits)
    out = np.empty(256, np.float32)
    n = lib().orc_materialize_block(P(a), a.size, block_idx, softcap, P(out))
    return out[:n]


class Rng:
    def __init__(self, seed):
        self.s = C.c_uint64(seed)

    def next_u64(self):
        return lib().orc_next_u64(C.byref(self.s))

    def next_f32(self):
        return lib().orc_next_f32(C.byref(self.s))

    @property
    def ref(self):
        return C.byref(self.s)


def dequantised_weights(cfg, weights, kind):
    """The fp32 weight set a quantised model actually multiplies with: every linear matrix goes
    through the oracle's quantise->de-quantise round trip (kind: "fp8" = e4m3 with a per-output-row
    scale, "int4" = 4-bit groups of 128 along the reduction axis); embeddings and norms stay as they
    are.  Also returns the out-major de-quantised matrices per layer (for bit-exact storage checks)."""
    L = lib()
    D, Q, KV, H = cfg.dim, cfg.q_dim, cfg.kv_dim, cfg.hidden

    def out_major(a, rows_in, cols_in, transpose):
        a = f32(a).reshape(rows_in, cols_in)
        return np.ascontiguousarray(a.T) if transpose else a

    def dq(m):
        m = np.ascontiguousarray(m, np.float32)
        out = np.empty_like(m)
        fn = L.orc_quant_fp8_rows if kind == "fp8" else L.orc_quant_int4_g128
        fn(P(m), m.shape[0], m.shape[1], None, None, P(out))
        return out

    shapes = dict(wq=(D, Q, True), wk=(D, KV, True), wv=(D, KV, True), wo=(Q, D, True), w1=(D, H, True),
                  w3=(D, H, True), w2=(D, H, False))
    out = {"embed": weights["embed"], "gamma_final": weights["gamma_final"], "layers": []}
    mats_per_layer = []
    for lw in weights["layers"]:
        mats = {n: dq(out_major(lw[n], *shape)) for n, shape in shapes.items()}
        lay = {n: np.ascontiguousarray(mats[n].T).ravel() for n in ("wq", "wk", "wv", "wo", "w1", "w3")}
        lay["w2"] = mats["w2"].ravel()
        lay["gamma1"], lay["gamma2"] = lw["gamma1"], lw["gamma2"]
        out["layers"].append(lay)
        mats_per_layer.append(mats)
    return out, mats_per_layer
