"""ctypes view of the C ABI in include/hip_decode.h.

Method names follow the reference's `metal_decode::Model` (crates/metal-decode/src/lib.rs:146-511)
so a test written against that type reads the same here.  Errors the reference raises as panics
come back as `HipDecodeError` carrying the status code.  There is no CPU fallback: if the library
is missing, importing a model fails.
"""
import ctypes as C
import enum
import os

import numpy as np

_LIB = None
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libhipdecode.so")

MAX_GPU_TOPK = 32
HEAD_BLOCK = 256

OK, ERR_ARG, ERR_FULL, ERR_HIP, ERR_UNSUPPORTED = 0, 1, 2, 3, 4

EXPORTS = [
    "hipdec_create", "hipdec_create_shared", "hipdec_create_packed", "hipdec_packed_sizes_of", "hipdec_export_packed_layer",
    "hipdec_export_packed_head", "hipdec_destroy", "hipdec_last_error", "hipdec_len", "hipdec_set_len", "hipdec_set_prefill_activations",
    "hipdec_seed_layer_cache_from_channel_first", "hipdec_decode_token", "hipdec_decode_token_from_id",
    "hipdec_decode_token_argmax", "hipdec_decode_token_argmax_from_id", "hipdec_decode_token_topk_from_id",
    "hipdec_decode_token_block_stats_from_id", "hipdec_materialize_current_logits_block",
    "hipdec_decode_logits_from_id", "hipdec_prefill", "hipdec_decode_greedy_run", "hipdec_last_device_ms",
    "hipdec_bytes_per_token", "hipdec_export_weight", "hipdec_debug_step_profile", "hipdec_debug_batch_step_profile", "hipdec_debug_calibration_copy",
    "hipdec_batch_begin", "hipdec_batch_end", "hipdec_batch_steps", "hipdec_batch_layers_in_one_launch", "hipdec_decode_logits_from_ids_batch",
    "hipdec_decode_token_argmax_from_ids_batch", "hipdec_decode_token_topk_from_ids_batch",
    "hipdec_decode_token_block_stats_from_ids_batch", "hipdec_materialize_current_logits_block_batch",
    "hipdec_decode_topk_sampled_run", "hipdec_decode_fullvocab_sampled_run", "hipdec_decode_topk_sampled_run_batch",
    "hipdec_decode_fullvocab_sampled_run_batch", "hipdec_debug_hostmath_eval", "hipdec_debug_hostmath_checksum",
    "hipdec_debug_hostmath_count_mismatch", "hipdec_debug_hostmath_probe", "hipdec_debug_sample_topk",
    "hipdec_debug_sample_fullvocab", "hipdec_sample_fullvocab_noalloc", "hipdec_debug_set_spin_limit", "hipdec_debug_step_kernel",
    "hipdec_debug_gemm_plan",
]


class WeightDtype(enum.IntEnum):
    F32 = 0
    BF16 = 1
    FP8_E4M3 = 2
    INT4_G128 = 3


class KvDtype(enum.IntEnum):
    F32 = 0
    BF16 = 1


class HipDecodeError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("hipdec status %d: %s" % (status, message))
        self.status = status


class Config(C.Structure):
    """metal_decode::Config, crates/metal-decode/src/lib.rs:22-35."""
    _fields_ = [(n, C.c_uint32) for n in
                ("dim", "hidden", "heads", "kv_heads", "hd", "seq", "nlayers", "vocab", "q_dim", "kv_dim", "gqa_ratio")]

    @classmethod
    def make(cls, dim, hidden, heads, hd, seq, nlayers, vocab, kv_heads=None):
        kv_heads = heads if kv_heads is None else kv_heads
        return cls(dim, hidden, heads, kv_heads, hd, seq, nlayers, vocab, heads * hd, kv_heads * hd, heads // kv_heads)

    def param_count(self):
        """ModelConfig::param_count, crates/engine/src/model.rs:182-187."""
        per_layer = 4 * self.dim * self.dim + 3 * self.dim * self.hidden
        return self.nlayers * per_layer + self.vocab * self.dim + self.dim * (2 * self.nlayers + 1)


class _Layer(C.Structure):
    _fields_ = [(n, C.POINTER(C.c_float)) for n in ("wq", "wk", "wv", "wo", "w1", "w3", "w2", "gamma1", "gamma2")]


class _Head(C.Structure):
    _fields_ = [("gamma_final", C.POINTER(C.c_float)), ("embed", C.POINTER(C.c_float))]


class _Options(C.Structure):
    _fields_ = [("weight_dtype", C.c_uint32), ("kv_dtype", C.c_uint32), ("device", C.c_int32),
                ("ffn_activation", C.c_uint32), ("flags", C.c_uint32), ("max_rows", C.c_uint32)]


FLAG_NO_GRAPH = 1


def load_library(path=None):
    """Loads libhipdecode.so (built in-tree by `__graft_entry__.build()`); raises if absent."""
    global _LIB
    if _LIB is not None and path is None:
        return _LIB
    p = path or _LIB_PATH
    if not os.path.exists(p):
        raise HipDecodeError(ERR_HIP, "%s not found: build it with __graft_entry__.build()" % p)
    lib = C.CDLL(p)
    lib.hipdec_last_error.restype = C.c_char_p
    lib.hipdec_last_error.argtypes = [C.c_void_p]
    lib.hipdec_len.restype = C.c_size_t
    lib.hipdec_len.argtypes = [C.c_void_p]
    lib.hipdec_destroy.restype = None
    lib.hipdec_destroy.argtypes = [C.c_void_p]
    fp, u32p = C.POINTER(C.c_float), C.POINTER(C.c_uint32)
    lib.hipdec_create.argtypes = [C.POINTER(Config), C.POINTER(_Layer), C.c_size_t, C.POINTER(_Head),
                                  C.POINTER(_Options), C.POINTER(C.c_void_p)]
    lib.hipdec_set_len.argtypes = [C.c_void_p, C.c_size_t]
    lib.hipdec_set_prefill_activations.argtypes = [C.c_void_p, C.c_int]
    lib.hipdec_seed_layer_cache_from_channel_first.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, fp, fp]
    lib.hipdec_decode_token.argtypes = [C.c_void_p, fp, fp]
    lib.hipdec_decode_token_from_id.argtypes = [C.c_void_p, C.c_uint32, fp]
    lib.hipdec_decode_token_argmax.argtypes = [C.c_void_p, fp, u32p]
    lib.hipdec_decode_token_argmax_from_id.argtypes = [C.c_void_p, C.c_uint32, u32p]
    lib.hipdec_decode_token_topk_from_id.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, fp, u32p, C.c_size_t,
                                                     C.POINTER(C.c_size_t)]
    lib.hipdec_decode_token_block_stats_from_id.argtypes = [C.c_void_p, C.c_uint32, C.c_float, C.c_float, fp, fp,
                                                            C.c_size_t, C.POINTER(C.c_size_t)]
    lib.hipdec_materialize_current_logits_block.argtypes = [C.c_void_p, C.c_size_t, C.c_float, fp, C.c_size_t,
                                                            C.POINTER(C.c_size_t)]
    lib.hipdec_decode_logits_from_id.argtypes = [C.c_void_p, C.c_uint32, C.c_float, fp]
    lib.hipdec_prefill.argtypes = [C.c_void_p, u32p, C.c_size_t, C.c_float, fp]
    lib.hipdec_decode_greedy_run.argtypes = [C.c_void_p, C.c_uint32, C.c_size_t, u32p]
    lib.hipdec_last_device_ms.argtypes = [C.c_void_p, fp]
    lib.hipdec_bytes_per_token.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(C.c_uint64)]
    lib.hipdec_export_weight.argtypes = [C.c_void_p, C.c_size_t, C.c_uint32, fp, C.c_size_t]
    lib.hipdec_debug_step_profile.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(C.c_uint64), C.c_size_t,
                                              C.POINTER(C.c_size_t)]
    lib.hipdec_debug_calibration_copy.argtypes = [C.c_size_t, C.c_int]
    szp = C.POINTER(C.c_size_t)
    lib.hipdec_batch_begin.argtypes = [C.c_void_p, C.c_size_t]
    lib.hipdec_batch_end.argtypes = [C.c_void_p]
    lib.hipdec_batch_steps.argtypes = [C.c_void_p, szp]
    lib.hipdec_decode_logits_from_ids_batch.argtypes = [C.c_void_p, u32p, C.c_float, fp]
    lib.hipdec_decode_token_argmax_from_ids_batch.argtypes = [C.c_void_p, u32p, u32p]
    lib.hipdec_decode_token_topk_from_ids_batch.argtypes = [C.c_void_p, u32p, C.c_uint32, fp, u32p, C.c_size_t, szp]
    lib.hipdec_decode_token_block_stats_from_ids_batch.argtypes = [C.c_void_p, u32p, C.c_float, C.c_float, fp, fp,
                                                                   C.c_size_t, szp]
    lib.hipdec_materialize_current_logits_block_batch.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_float, fp,
                                                                  C.c_size_t, szp]
    u64p = C.POINTER(C.c_uint64)
    lib.hipdec_decode_topk_sampled_run.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_float, C.c_float, u64p,
                                                   C.c_size_t, u32p]
    lib.hipdec_decode_fullvocab_sampled_run.argtypes = [C.c_void_p, C.c_uint32, C.c_float, C.c_float, u64p, C.c_size_t,
                                                        u32p]
    lib.hipdec_decode_topk_sampled_run_batch.argtypes = [C.c_void_p, u32p, C.c_uint32, C.c_float, C.c_float, u64p,
                                                         C.c_size_t, u32p]
    lib.hipdec_decode_fullvocab_sampled_run_batch.argtypes = [C.c_void_p, u32p, C.c_float, C.c_float, u64p, C.c_size_t,
                                                              u32p]
    lib.hipdec_debug_hostmath_eval.argtypes = [C.c_int, fp, fp, C.c_size_t, C.c_int]
    lib.hipdec_debug_hostmath_checksum.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_int, C.c_int, u64p]
    lib.hipdec_debug_hostmath_count_mismatch.argtypes = [C.c_int, C.c_uint32, C.c_uint64, C.c_int, u64p]
    lib.hipdec_debug_sample_topk.argtypes = [fp, u32p, C.c_size_t, C.c_uint32, C.c_float, C.c_float, u64p, u32p]
    lib.hipdec_debug_sample_fullvocab.argtypes = [fp, C.c_size_t, fp, fp, C.c_float, C.c_float, u64p, u32p]
    lib.hipdec_sample_fullvocab_noalloc.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_float, C.c_float,
                                                    C.c_void_p, C.c_void_p, C.c_void_p]
    if path is None:
        _LIB = lib
    return lib


HOSTMATH_EXPF, HOSTMATH_TANHF = 0, 1


def debug_hostmath(fn, x, on_device=False):
    """The sampler's restatement of the host C library's expf (fn 0) or tanhf (fn 1), evaluated on
    the host or on the GPU."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    rc = load_library().hipdec_debug_hostmath_eval(fn, _fptr(x), _fptr(out), x.size, 1 if on_device else 0)
    if rc != OK:
        raise HipDecodeError(rc, "hipdec_debug_hostmath_eval failed")
    return out


def debug_hostmath_checksum(fn, first_bits, count, on_device=False, host_threads=8):
    out = C.c_uint64()
    rc = load_library().hipdec_debug_hostmath_checksum(fn, first_bits, count, 1 if on_device else 0, host_threads,
                                                       C.byref(out))
    if rc != OK:
        raise HipDecodeError(rc, "hipdec_debug_hostmath_checksum failed")
    return out.value


def debug_hostmath_count_mismatch(fn, first_bits, count, host_threads=8):
    """How many of `count` consecutive float bit patterns give a result different from libm's function."""
    out = C.c_uint64()
    rc = load_library().hipdec_debug_hostmath_count_mismatch(fn, first_bits, count, host_threads, C.byref(out))
    if rc != OK:
        raise HipDecodeError(rc, "hipdec_debug_hostmath_count_mismatch failed")
    return out.value


def debug_sample_topk(vals, idxs, top_k, temperature, rng_state, softcap=0.0):
    """The on-device merge + draw over per-block candidate lists [blocks * top_k]; returns (token, new state)."""
    v = np.ascontiguousarray(vals, dtype=np.float32)
    i = np.ascontiguousarray(idxs, dtype=np.uint32)
    st, tok = C.c_uint64(int(rng_state) & 0xFFFFFFFFFFFFFFFF), C.c_uint32()
    rc = load_library().hipdec_debug_sample_topk(_fptr(v), i.ctypes.data_as(C.POINTER(C.c_uint32)), v.size // top_k, top_k,
                                                 temperature, softcap, C.byref(st), C.byref(tok))
    if rc != OK:
        raise HipDecodeError(rc, "hipdec_debug_sample_topk failed")
    return tok.value, st.value


def debug_sample_fullvocab(logits, maxes, sums, temperature, rng_state, softcap=0.0):
    """The on-device block draw + token draw over raw logits and their block statistics; returns (token, new state)."""
    lg, mx, sm = (np.ascontiguousarray(a, dtype=np.float32) for a in (logits, maxes, sums))
    st, tok = C.c_uint64(int(rng_state) & 0xFFFFFFFFFFFFFFFF), C.c_uint32()
    rc = load_library().hipdec_debug_sample_fullvocab(_fptr(lg), lg.size, _fptr(mx), _fptr(sm), temperature, softcap,
                                                      C.byref(st), C.byref(tok))
    if rc != OK:
        raise HipDecodeError(rc, "hipdec_debug_sample_fullvocab failed")
    return tok.value, st.value


def sample_fullvocab_noalloc(d_logits, vocab, d_maxes, d_sums, temperature, d_rng_state, d_out_token, softcap=0.0,
                             stream=None):
    """hipdec_sample_fullvocab_noalloc: every pointer is a device address (an int); enqueues on `stream`
    (a hipStream_t as an int, None = default stream) and returns without waiting."""
    rc = load_library().hipdec_sample_fullvocab_noalloc(d_logits, vocab, d_maxes, d_sums, temperature, softcap,
                                                        d_rng_state, d_out_token, stream)
    if rc != OK:
        raise HipDecodeError(rc, (load_library().hipdec_last_error(None) or b"").decode())


def calibration_copy(nbytes, reps=1):
    """Runs the plain copy kernel (k_calib_copy) of a known size: the yardstick for traffic counters."""
    rc = load_library().hipdec_debug_calibration_copy(nbytes, reps)
    if rc != OK:
        raise HipDecodeError(rc, "calibration copy failed")


def set_spin_limit(check_mask=127, limit=1 << 22):
    """Test hook: how the persistent kernels bound their waits (hipdec_debug_set_spin_limit); the defaults restore them."""
    lib = load_library()
    lib.hipdec_debug_set_spin_limit.argtypes = [C.c_uint32, C.c_uint32]
    rc = lib.hipdec_debug_set_spin_limit(check_mask, limit)
    if rc != OK:
        raise HipDecodeError(rc, (lib.hipdec_last_error(None) or b"").decode())


GEMM_KERNELS = ("tiled", "tiled_direct_lds", "few_row", "few_row_int4", "few_row_e4m3")


def gemm_plan(weight_dtype, rows, n, k, num_cu=256):
    """The launch the library uses for the product of `rows` activation rows with an [n][k] weight matrix
    (hipdec_debug_gemm_plan; host arithmetic only, no GPU needed)."""
    lib = load_library()
    out = (C.c_uint64 * 8)()
    lib.hipdec_debug_gemm_plan.argtypes = [C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_uint64)]
    rc = lib.hipdec_debug_gemm_plan(int(weight_dtype), rows, n, k, num_cu, out)
    if rc != OK:
        raise HipDecodeError(rc, "the library launches no such product")
    return {"kernel": GEMM_KERNELS[out[0]], "splits": out[1], "steps_per_split": out[2], "grid": (out[3], out[4], out[5]),
            "threads": out[6], "lds_bytes": out[7]}


def _fptr(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _f32(a, n=None, name="array"):
    a = np.ascontiguousarray(a, dtype=np.float32)
    if n is not None and a.size != n:
        raise ValueError("%s has %d elements, expected %d" % (name, a.size, n))
    return a


class HipDecodeModel:
    """`metal_decode::Model` over the HIP backend.

    weights: dict with "embed" [vocab*dim], "gamma_final" [dim] and "layers": list of dicts with
    wq wk wv wo w1 w3 w2 gamma1 gamma2 in the reference's layouts (crates/engine/src/layer.rs:19-36).
    """

    def __init__(self, cfg, weights, weight_dtype=WeightDtype.F32, kv_dtype=KvDtype.F32, device=0,
                 ffn_activation=0, flags=0):
        self._lib = load_library()
        self._h = C.c_void_p()
        self.cfg = cfg
        D, Q, KV, H, V = cfg.dim, cfg.q_dim, cfg.kv_dim, cfg.hidden, cfg.vocab
        sizes = dict(wq=D * Q, wk=D * KV, wv=D * KV, wo=Q * D, w1=D * H, w3=D * H, w2=D * H, gamma1=D, gamma2=D)
        keep = []
        layers = (_Layer * len(weights["layers"]))()
        for i, lw in enumerate(weights["layers"]):
            for name, n in sizes.items():
                a = _f32(lw[name], n, name)
                keep.append(a)
                setattr(layers[i], name, _fptr(a))
        embed = _f32(weights["embed"], V * D, "embed")
        gf = _f32(weights["gamma_final"], D, "gamma_final")
        head = _Head(_fptr(gf), _fptr(embed))
        opts = _Options(int(weight_dtype), int(kv_dtype), device, ffn_activation, flags, 0)
        rc = self._lib.hipdec_create(C.byref(cfg), layers, len(weights["layers"]), C.byref(head), C.byref(opts),
                                     C.byref(self._h))
        if rc != OK:
            raise HipDecodeError(rc, (self._lib.hipdec_last_error(None) or b"").decode())
        self.blocks = (V + HEAD_BLOCK - 1) // HEAD_BLOCK
        self._rows = 0

    def create_shared(self, kv_dtype=KvDtype.F32, flags=0):
        """A second model on this model's device weights (no upload): own KV caches and step state."""
        other = object.__new__(HipDecodeModel)
        other._lib = self._lib
        other._h = C.c_void_p()
        other.cfg = self.cfg
        self._lib.hipdec_create_shared.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(C.c_void_p)]
        rc = self._lib.hipdec_create_shared(self._h, int(kv_dtype), int(flags), C.byref(other._h))
        if rc != OK:
            raise HipDecodeError(rc, (self._lib.hipdec_last_error(None) or b"").decode())
        other.blocks = self.blocks
        other._rows = 0
        return other

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            self._lib.hipdec_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _chk(self, rc):
        if rc != OK:
            raise HipDecodeError(rc, (self._lib.hipdec_last_error(self._h) or b"").decode())

    # ---- metal_decode::Model surface
    def len(self):
        return int(self._lib.hipdec_len(self._h))

    def set_len(self, n):
        self._chk(self._lib.hipdec_set_len(self._h, n))

    def set_prefill_activations(self, mode):
        """How the prefill GEMMs take their activations: 0 the (hi, lo) bf16 pair, 1 one bf16 number, 2 one fp16 number."""
        self._chk(self._lib.hipdec_set_prefill_activations(self._h, int(mode)))

    def seed_layer_cache_from_channel_first(self, layer_idx, live_len, k_rope_cf, v_cf):
        n = self.cfg.kv_dim * self.cfg.seq
        k, v = _f32(k_rope_cf, n, "k_rope_cf"), _f32(v_cf, n, "v_cf")
        self._chk(self._lib.hipdec_seed_layer_cache_from_channel_first(self._h, layer_idx, live_len, _fptr(k), _fptr(v)))

    def decode_token(self, x_in):
        x = _f32(x_in, self.cfg.dim, "x_in")
        out = np.empty(self.cfg.dim, np.float32)
        self._chk(self._lib.hipdec_decode_token(self._h, _fptr(x), _fptr(out)))
        return out

    def decode_token_from_id(self, token):
        out = np.empty(self.cfg.dim, np.float32)
        self._chk(self._lib.hipdec_decode_token_from_id(self._h, token, _fptr(out)))
        return out

    def decode_token_argmax(self, x_in):
        x = _f32(x_in, self.cfg.dim, "x_in")
        t = C.c_uint32()
        self._chk(self._lib.hipdec_decode_token_argmax(self._h, _fptr(x), C.byref(t)))
        return t.value

    def step_kernel(self):
        """0: one kernel per product, 1: the persistent step kernel, 2: its short-phase form (hipdec_debug_step_kernel)."""
        v = C.c_int()
        self._lib.hipdec_debug_step_kernel.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
        self._chk(self._lib.hipdec_debug_step_kernel(self._h, C.byref(v)))
        return v.value

    def decode_token_argmax_from_id(self, token):
        t = C.c_uint32()
        self._chk(self._lib.hipdec_decode_token_argmax_from_id(self._h, token, C.byref(t)))
        return t.value

    def decode_token_topk_from_id(self, token, top_k, cap=None):
        cap = self.blocks * max(int(top_k), 1) if cap is None else cap
        vals = np.empty(max(cap, 1), np.float32)
        idxs = np.empty(max(cap, 1), np.uint32)
        cnt = C.c_size_t()
        self._chk(self._lib.hipdec_decode_token_topk_from_id(
            self._h, token, top_k, _fptr(vals), idxs.ctypes.data_as(C.POINTER(C.c_uint32)), cap, C.byref(cnt)))
        return vals[:cnt.value], idxs[:cnt.value]

    def decode_token_block_stats_from_id(self, token, inv_temperature, softcap, cap=None):
        cap = self.blocks if cap is None else cap
        mx = np.empty(max(cap, 1), np.float32)
        sm = np.empty(max(cap, 1), np.float32)
        cnt = C.c_size_t()
        self._chk(self._lib.hipdec_decode_token_block_stats_from_id(
            self._h, token, inv_temperature, softcap, _fptr(mx), _fptr(sm), cap, C.byref(cnt)))
        return mx[:cnt.value], sm[:cnt.value]

    def materialize_current_logits_block(self, block_idx, softcap, cap=HEAD_BLOCK):
        out = np.empty(max(cap, 1), np.float32)
        valid = C.c_size_t()
        self._chk(self._lib.hipdec_materialize_current_logits_block(self._h, block_idx, softcap, _fptr(out), cap,
                                                                    C.byref(valid)))
        return out[:valid.value]

    # ---- additions
    def decode_logits_from_id(self, token, softcap=0.0):
        out = np.empty(self.cfg.vocab, np.float32)
        self._chk(self._lib.hipdec_decode_logits_from_id(self._h, token, softcap, _fptr(out)))
        return out

    def prefill(self, ids, softcap=0.0, want_logits=True):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        out = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        self._chk(self._lib.hipdec_prefill(self._h, ids.ctypes.data_as(C.POINTER(C.c_uint32)), ids.size, softcap,
                                           _fptr(out) if want_logits else None))
        return out

    def decode_greedy_run(self, token, n_steps):
        out = np.empty(max(n_steps, 1), np.uint32)
        self._chk(self._lib.hipdec_decode_greedy_run(self._h, token, n_steps,
                                                     out.ctypes.data_as(C.POINTER(C.c_uint32))))
        return out[:n_steps]

    # ---- sampled runs with the draw on the device; return (tokens, new rng state)
    def decode_topk_sampled_run(self, token, top_k, temperature, rng_state, n_steps, softcap=0.0):
        out = np.empty(max(n_steps, 1), np.uint32)
        st = C.c_uint64(int(rng_state) & 0xFFFFFFFFFFFFFFFF)
        self._chk(self._lib.hipdec_decode_topk_sampled_run(self._h, token, top_k, temperature, softcap, C.byref(st),
                                                           n_steps, out.ctypes.data_as(C.POINTER(C.c_uint32))))
        return out[:n_steps], st.value

    def decode_fullvocab_sampled_run(self, token, temperature, rng_state, n_steps, softcap=0.0):
        out = np.empty(max(n_steps, 1), np.uint32)
        st = C.c_uint64(int(rng_state) & 0xFFFFFFFFFFFFFFFF)
        self._chk(self._lib.hipdec_decode_fullvocab_sampled_run(self._h, token, temperature, softcap, C.byref(st),
                                                                n_steps, out.ctypes.data_as(C.POINTER(C.c_uint32))))
        return out[:n_steps], st.value

    def decode_topk_sampled_run_batch(self, tokens, top_k, temperature, rng_states, n_steps, softcap=0.0):
        t = self._toks(tokens)
        st = np.ascontiguousarray(rng_states, dtype=np.uint64).copy()
        if st.size != self._rows:
            raise ValueError("expected %d rng states, got %d" % (self._rows, st.size))
        out = np.empty((max(n_steps, 1), self._rows), np.uint32)
        self._chk(self._lib.hipdec_decode_topk_sampled_run_batch(
            self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)), top_k, temperature, softcap,
            st.ctypes.data_as(C.POINTER(C.c_uint64)), n_steps, out.ctypes.data_as(C.POINTER(C.c_uint32))))
        return out[:n_steps], st

    def decode_fullvocab_sampled_run_batch(self, tokens, temperature, rng_states, n_steps, softcap=0.0):
        t = self._toks(tokens)
        st = np.ascontiguousarray(rng_states, dtype=np.uint64).copy()
        if st.size != self._rows:
            raise ValueError("expected %d rng states, got %d" % (self._rows, st.size))
        out = np.empty((max(n_steps, 1), self._rows), np.uint32)
        self._chk(self._lib.hipdec_decode_fullvocab_sampled_run_batch(
            self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)), temperature, softcap,
            st.ctypes.data_as(C.POINTER(C.c_uint64)), n_steps, out.ctypes.data_as(C.POINTER(C.c_uint32))))
        return out[:n_steps], st

    # ---- multi-sample decode: rows share positions [0, len) and step together
    def batch_begin(self, n_rows):
        self._chk(self._lib.hipdec_batch_begin(self._h, n_rows))
        self._rows = int(n_rows)

    def batch_end(self):
        self._chk(self._lib.hipdec_batch_end(self._h))
        self._rows = 0

    def batch_layers_in_one_launch(self):
        v = C.c_int()
        self._chk(self._lib.hipdec_batch_layers_in_one_launch(self._h, C.byref(v)))
        return bool(v.value)

    def debug_batch_step_profile(self, tokens):
        """Time stamps of workgroup 0 for one step of the open batch: array [nlayers + 1][16] of 100 MHz ticks."""
        t = self._toks(tokens)
        n = (self.cfg.nlayers + 1) * 16
        out = np.zeros(n, np.uint64)
        cnt = C.c_size_t()
        self._chk(self._lib.hipdec_debug_batch_step_profile(self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)),
                                                            out.ctypes.data_as(C.POINTER(C.c_uint64)), n, C.byref(cnt)))
        return out.reshape(self.cfg.nlayers + 1, 16)

    def batch_steps(self):
        n = C.c_size_t()
        self._chk(self._lib.hipdec_batch_steps(self._h, C.byref(n)))
        return n.value

    def _toks(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        if t.size != self._rows:
            raise ValueError("expected %d tokens, got %d" % (self._rows, t.size))
        return t

    def decode_logits_from_ids_batch(self, tokens, softcap=0.0):
        t = self._toks(tokens)
        out = np.empty((self._rows, self.cfg.vocab), np.float32)
        self._chk(self._lib.hipdec_decode_logits_from_ids_batch(self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)), softcap,
                                                               _fptr(out)))
        return out

    def decode_token_argmax_from_ids_batch(self, tokens):
        t = self._toks(tokens)
        out = np.empty(self._rows, np.uint32)
        self._chk(self._lib.hipdec_decode_token_argmax_from_ids_batch(
            self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)), out.ctypes.data_as(C.POINTER(C.c_uint32))))
        return out

    def decode_token_topk_from_ids_batch(self, tokens, top_k):
        t = self._toks(tokens)
        per = self.blocks * max(int(top_k), 1)
        vals = np.empty((self._rows, per), np.float32)
        idxs = np.empty((self._rows, per), np.uint32)
        cnt = C.c_size_t()
        self._chk(self._lib.hipdec_decode_token_topk_from_ids_batch(
            self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)), top_k, _fptr(vals),
            idxs.ctypes.data_as(C.POINTER(C.c_uint32)), vals.size, C.byref(cnt)))
        return vals, idxs

    def decode_token_block_stats_from_ids_batch(self, tokens, inv_temperature, softcap):
        t = self._toks(tokens)
        mx = np.empty((self._rows, self.blocks), np.float32)
        sm = np.empty((self._rows, self.blocks), np.float32)
        cnt = C.c_size_t()
        self._chk(self._lib.hipdec_decode_token_block_stats_from_ids_batch(
            self._h, t.ctypes.data_as(C.POINTER(C.c_uint32)), inv_temperature, softcap, _fptr(mx), _fptr(sm), mx.size,
            C.byref(cnt)))
        return mx, sm

    def materialize_current_logits_block_batch(self, row, block_idx, softcap, cap=HEAD_BLOCK):
        out = np.empty(max(cap, 1), np.float32)
        valid = C.c_size_t()
        self._chk(self._lib.hipdec_materialize_current_logits_block_batch(self._h, row, block_idx, softcap, _fptr(out),
                                                                          cap, C.byref(valid)))
        return out[:valid.value]

    def last_device_ms(self):
        ms = C.c_float()
        self._chk(self._lib.hipdec_last_device_ms(self._h, C.byref(ms)))
        return ms.value

    def bytes_per_token(self, kv_len):
        b = C.c_uint64()
        self._chk(self._lib.hipdec_bytes_per_token(self._h, kv_len, C.byref(b)))
        return b.value

    def debug_step_profile(self, token):
        n = (self.cfg.nlayers + 1) * 32
        out = np.zeros(n, np.uint64)
        cnt = C.c_size_t()
        self._chk(self._lib.hipdec_debug_step_profile(self._h, token, out.ctypes.data_as(C.POINTER(C.c_uint64)), n,
                                                      C.byref(cnt)))
        return out.reshape(self.cfg.nlayers + 1, 32)

    def export_weight(self, layer_idx, which):
        c = self.cfg
        shapes = {0: (c.q_dim + 2 * c.kv_dim, c.dim), 1: (c.dim, c.q_dim), 2: (2 * c.hidden, c.dim),
                  3: (c.dim, c.hidden), 4: (c.vocab, c.dim)}
        rows, k = shapes[which]
        out = np.empty(rows * k, np.float32)
        self._chk(self._lib.hipdec_export_weight(self._h, layer_idx, which, _fptr(out), out.size))
        return out.reshape(rows, k)
