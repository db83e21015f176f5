"""ctypes view of the host engine (librustane_engine.so): the session API of the reference's
`engine::inference` (crates/engine/src/inference.rs) over the HIP decode backend, its samplers and
its backend selection.  Names follow the reference."""
import ctypes as C
import enum

import numpy as np

from .synth import load_engine

fp = C.POINTER(C.c_float)
u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)

AUTO_KV_PARAM_THRESHOLD = 20_000_000       # inference.rs:9
MAX_GPU_TOPK = 32


class DecodeBackendRequest(enum.IntEnum):
    AUTO = 0
    NAIVE = 1
    HIP = 2


class DecodeMode(enum.IntEnum):
    PREFILL_ONLY = 0
    NAIVE_FULL_CONTEXT = 1
    KV_CACHE_HIP = 2


class RsConfig(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("dim", "hidden", "heads", "kv_heads", "hd", "seq", "nlayers", "vocab")] + \
               [("ffn_activation", C.c_uint32)]

    @classmethod
    def of(cls, cfg, ffn_activation=0):
        return cls(cfg.dim, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.hd, cfg.seq, cfg.nlayers, cfg.vocab,
                   ffn_activation)


class RsRequest(C.Structure):
    _fields_ = [("backend", C.c_uint32), ("steps", C.c_uint64), ("temperature", C.c_float), ("top_k", C.c_uint64),
                ("samples", C.c_uint64), ("seed", C.c_uint64)]


class RsBatchInfo(C.Structure):
    _fields_ = [("mode", C.c_uint32), ("fallback_reason", C.c_char_p), ("auto_reason", C.c_char_p),
                ("base_prefill_s", C.c_double), ("request_prefill_s", C.c_double), ("prefill_s", C.c_double),
                ("total_decode_s", C.c_double), ("avg_decode_s", C.c_double), ("total_s", C.c_double),
                ("n_results", C.c_uint64)]


_bound = False


def lib():
    global _bound
    L = load_engine()
    if not _bound:
        L.rs_param_count.restype = C.c_uint64
        L.rs_param_count.argtypes = [C.POINTER(RsConfig)]
        L.rs_weights_synthetic.restype = C.c_void_p
        L.rs_weights_synthetic.argtypes = [C.POINTER(RsConfig), C.c_uint64, C.c_float, C.c_int]
        L.rs_weights_from_arrays.restype = C.c_void_p
        L.rs_weights_from_arrays.argtypes = [C.POINTER(RsConfig), C.POINTER(fp), fp, fp]
        L.rs_weights_free.argtypes = [C.c_void_p]
        L.rs_checkpoint_parse.restype = C.c_void_p
        L.rs_checkpoint_parse.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(RsConfig), u32p, C.c_char_p, C.c_size_t]
        L.rs_checkpoint_load.restype = C.c_void_p
        L.rs_checkpoint_load.argtypes = [C.c_char_p, C.POINTER(RsConfig), u32p, C.c_char_p, C.c_size_t]
        L.rs_checkpoint_write.argtypes = [C.c_char_p, C.POINTER(RsConfig), C.c_void_p, C.c_uint32, C.c_char_p, C.c_size_t]
        L.rs_jsonl_parse.argtypes = [C.c_char_p, C.POINTER(RsRequest), C.POINTER(RsRequest), u32p, C.c_size_t, u64p,
                                     C.c_char_p, C.c_size_t]
        L.rs_http_parse_request.argtypes = [C.c_int, C.c_uint64, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_char_p,
                                            C.c_size_t, u64p, C.c_char_p, C.c_size_t]
        L.rs_http_prepare.argtypes = [C.c_char_p, C.c_int, C.c_char_p, C.c_uint64, C.c_uint32, C.POINTER(RsRequest),
                                      C.POINTER(C.c_int), u32p, C.c_size_t, u64p, C.c_char_p, C.c_size_t]
        L.rs_http_render_chat_prompt.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]
        L.rs_packed_checkpoint_parse.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(RsConfig), u32p, u32p, C.c_char_p, C.c_size_t]
        L.rs_weights_tensor.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.POINTER(fp), u64p]
        L.rs_session_new.restype = C.c_void_p
        L.rs_session_new.argtypes = [C.POINTER(RsConfig), C.c_void_p, u32p, C.c_size_t, C.c_float, C.c_uint32,
                                     C.c_uint32, C.c_uint32, C.c_char_p, C.c_size_t]
        L.rs_session_free.argtypes = [C.c_void_p]
        L.rs_session_prompt_len.restype = C.c_uint64
        L.rs_session_prompt_len.argtypes = [C.c_void_p]
        L.rs_session_prefill_s.restype = C.c_double
        L.rs_session_prefill_s.argtypes = [C.c_void_p]
        L.rs_session_prompt_logits.argtypes = [C.c_void_p, fp]
        L.rs_session_generate.argtypes = [C.c_void_p, C.POINTER(RsRequest), u32p, C.c_size_t, C.c_int, C.c_uint64,
                                          C.POINTER(RsBatchInfo), C.c_char_p, C.c_size_t]
        L.rs_session_batch_device_ms.restype = C.c_double
        L.rs_session_batch_device_ms.argtypes = [C.c_void_p]
        L.rs_session_bytes_per_token.restype = C.c_uint64
        L.rs_session_bytes_per_token.argtypes = [C.c_void_p, C.c_size_t]
        L.rs_session_stream_count.restype = C.c_uint64
        L.rs_session_stream_count.argtypes = [C.c_void_p]
        L.rs_session_result_len.restype = C.c_uint64
        L.rs_session_result_len.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
        L.rs_session_result_copy.argtypes = [C.c_void_p, C.c_size_t, C.c_int, u32p]
        L.rs_session_result_decode_s.restype = C.c_double
        L.rs_session_result_decode_s.argtypes = [C.c_void_p, C.c_size_t]
        L.rs_session_result_seed.restype = C.c_uint64
        L.rs_session_result_seed.argtypes = [C.c_void_p, C.c_size_t]
        L.rs_session_cache_new.restype = C.c_void_p
        L.rs_session_cache_new.argtypes = [C.POINTER(RsConfig), C.c_void_p, C.c_float, C.c_size_t, C.c_uint32, C.c_uint32,
                                           C.c_uint32]
        L.rs_session_cache_free.argtypes = [C.c_void_p]
        L.rs_session_cache_len.restype = C.c_uint64
        L.rs_session_cache_len.argtypes = [C.c_void_p]
        L.rs_session_cache_max_entries.restype = C.c_uint64
        L.rs_session_cache_max_entries.argtypes = [C.c_void_p]
        L.rs_session_cache_entry_prompt.restype = C.c_uint64
        L.rs_session_cache_entry_prompt.argtypes = [C.c_void_p, C.c_size_t, u32p, C.c_size_t]
        L.rs_session_cache_normalize.restype = C.c_uint64
        L.rs_session_cache_normalize.argtypes = [C.c_void_p, u32p, C.c_size_t, u32p, C.c_size_t]
        L.rs_session_cache_find.restype = C.c_int64
        L.rs_session_cache_find.argtypes = [C.c_void_p, u32p, C.c_size_t, C.c_int]
        L.rs_session_cache_insert.restype = C.c_int64
        L.rs_session_cache_insert.argtypes = [C.c_void_p, u32p, C.c_size_t, C.c_char_p, C.c_size_t]
        L.rs_session_cache_generate.argtypes = [C.c_void_p, u32p, C.c_size_t, C.POINTER(RsRequest), C.c_int, C.c_uint64,
                                                C.POINTER(RsBatchInfo), u64p, C.c_char_p, C.c_size_t]
        L.rs_session_cache_result_len.restype = C.c_uint64
        L.rs_session_cache_result_len.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
        L.rs_session_cache_result_copy.argtypes = [C.c_void_p, C.c_size_t, C.c_int, u32p]
        L.rs_session_cache_result_seed.restype = C.c_uint64
        L.rs_session_cache_result_seed.argtypes = [C.c_void_p, C.c_size_t]
        L.rs_select_decode_mode.argtypes = [C.POINTER(RsConfig), C.c_uint32, C.c_uint64, C.c_uint64, u32p,
                                            C.POINTER(C.c_char_p), C.POINTER(C.c_char_p)]
        L.rs_parse_decode_backend.argtypes = [C.c_char_p, u32p]
        L.rs_next_u64.restype = C.c_uint64
        L.rs_next_u64.argtypes = [u64p]
        L.rs_next_f32.restype = C.c_float
        L.rs_next_f32.argtypes = [u64p]
        L.rs_sample_next.restype = C.c_uint32
        L.rs_sample_next.argtypes = [fp, C.c_size_t, C.c_float, C.c_size_t, u64p]
        L.rs_sample_topk_candidates.restype = C.c_uint32
        L.rs_sample_topk_candidates.argtypes = [u32p, fp, C.c_size_t, C.c_float, u64p]
        L.rs_sample_block_from_stats.restype = C.c_uint64
        L.rs_sample_block_from_stats.argtypes = [fp, fp, C.c_size_t, u64p]
        L.rs_sample_softmax_index.restype = C.c_uint64
        L.rs_sample_softmax_index.argtypes = [fp, C.c_size_t, C.c_float, u64p]
        L.rs_sample_block_logits.restype = C.c_uint32
        L.rs_sample_block_logits.argtypes = [C.c_uint32, fp, C.c_size_t, C.c_float, u64p]
        L.rs_merge_topk_candidates.restype = C.c_uint64
        L.rs_merge_topk_candidates.argtypes = [fp, u32p, C.c_size_t, C.c_size_t, fp, u32p]
        L.rs_validate_token_ids.argtypes = [u32p, C.c_size_t, C.c_size_t, C.c_char_p, C.c_char_p, C.c_size_t]
        L.rs_fill_input_window.restype = C.c_uint64
        L.rs_fill_input_window.argtypes = [u32p, C.c_size_t, C.c_size_t, u32p]
        _bound = True
    return L


def param_count(cfg):
    return lib().rs_param_count(C.byref(RsConfig.of(cfg)))


def parse_decode_backend(raw):
    out = C.c_uint32()
    return DecodeBackendRequest(out.value) if lib().rs_parse_decode_backend(raw.encode(), C.byref(out)) else None


class DecodeSelection:
    def __init__(self, mode, fallback_reason, auto_reason):
        self.mode = DecodeMode(mode)
        self.fallback_reason = fallback_reason.decode() if fallback_reason else None
        self.auto_reason = auto_reason.decode() if auto_reason else None


def select_decode_mode(cfg, requested, effective_context_len, steps):
    """inference.rs:458-528."""
    mode = C.c_uint32()
    fb, ar = C.c_char_p(), C.c_char_p()
    lib().rs_select_decode_mode(C.byref(RsConfig.of(cfg)), int(requested), effective_context_len, steps,
                                C.byref(mode), C.byref(fb), C.byref(ar))
    return DecodeSelection(mode.value, fb.value, ar.value)


class GenerationRequest:
    """inference.rs:61-82 (same defaults)."""

    def __init__(self, decode_backend=DecodeBackendRequest.AUTO, steps=32, temperature=0.0, top_k=0, samples=1, seed=1):
        self.decode_backend, self.steps, self.temperature = decode_backend, steps, temperature
        self.top_k, self.samples, self.seed = top_k, samples, seed

    def _c(self):
        return RsRequest(int(self.decode_backend), self.steps, self.temperature, self.top_k, self.samples, self.seed)


class SampleResult:
    def __init__(self, seed, generated, sampled, decode_elapsed):
        self.seed, self.generated, self.sampled, self.decode_elapsed = seed, generated, sampled, decode_elapsed


class GenerationBatch:
    def __init__(self, info, results):
        self.decode_selection = DecodeSelection(info.mode, info.fallback_reason, info.auto_reason)
        self.base_prefill_elapsed = info.base_prefill_s
        self.request_prefill_elapsed = info.request_prefill_s
        self.prefill_elapsed = info.prefill_s
        self.total_decode_elapsed = info.total_decode_s
        self.avg_decode_elapsed = info.avg_decode_s
        self.total_elapsed = info.total_s
        self.results = results


class SessionError(RuntimeError):
    pass


class InferenceSession:
    """inference.rs:107-452 over the HIP backend.  weights: the dict layout of rustane_amd.synth.make_weights."""

    def __init__(self, cfg, weights, prompt_ids, softcap=0.0, weight_dtype=0, kv_dtype=0, flags=0, ffn_activation=0):
        L = lib()
        self._L = L
        self.cfg = cfg
        rc = RsConfig.of(cfg, ffn_activation)
        names = ("wq", "wk", "wv", "wo", "w1", "w3", "w2", "gamma1", "gamma2")
        keep, ptrs = [], (fp * (9 * cfg.nlayers))()
        for l, lw in enumerate(weights["layers"]):
            for k, nme in enumerate(names):
                a = np.ascontiguousarray(lw[nme], np.float32)
                keep.append(a)
                ptrs[l * 9 + k] = a.ctypes.data_as(fp)
        gf = np.ascontiguousarray(weights["gamma_final"], np.float32)
        em = np.ascontiguousarray(weights["embed"], np.float32)
        self._w = C.c_void_p(L.rs_weights_from_arrays(C.byref(rc), ptrs, gf.ctypes.data_as(fp), em.ctypes.data_as(fp)))
        ids = np.ascontiguousarray(prompt_ids, np.uint32)
        err = C.create_string_buffer(512)
        self._s = C.c_void_p(L.rs_session_new(C.byref(rc), self._w, ids.ctypes.data_as(u32p), ids.size, softcap,
                                              int(weight_dtype), int(kv_dtype), flags, err, 512))
        if not self._s.value:
            L.rs_weights_free(self._w)
            self._w = None
            raise SessionError(err.value.decode())

    def close(self):
        if getattr(self, "_s", None) and self._s.value:
            self._L.rs_session_free(self._s)
            self._s = C.c_void_p()
        if getattr(self, "_w", None):
            self._L.rs_weights_free(self._w)
            self._w = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def prompt_len(self):
        return int(self._L.rs_session_prompt_len(self._s))

    def prefill_elapsed(self):
        return self._L.rs_session_prefill_s(self._s)

    def prompt_logits(self):
        out = np.empty(self.cfg.vocab, np.float32)
        self._L.rs_session_prompt_logits(self._s, out.ctypes.data_as(fp))
        return out

    def _run(self, req, suffix, stream, abort_after):
        suf = np.ascontiguousarray(suffix, np.uint32)
        info = RsBatchInfo()
        err = C.create_string_buffer(512)
        rc = self._L.rs_session_generate(self._s, C.byref(req._c()), suf.ctypes.data_as(u32p), suf.size, int(stream),
                                         abort_after, C.byref(info), err, 512)
        if rc:
            raise SessionError(err.value.decode())
        results = []
        for i in range(info.n_results):
            arrs = []
            for which in (0, 1):
                n = self._L.rs_session_result_len(self._s, i, which)
                a = np.empty(max(n, 1), np.uint32)
                self._L.rs_session_result_copy(self._s, i, which, a.ctypes.data_as(u32p))
                arrs.append(a[:n])
            results.append(SampleResult(self._L.rs_session_result_seed(self._s, i), arrs[1], arrs[0],
                                        self._L.rs_session_result_decode_s(self._s, i)))
        return GenerationBatch(info, results)

    def generate(self, req):
        return self._run(req, (), False, 0)

    def generate_with_suffix(self, req, prompt_suffix):
        return self._run(req, prompt_suffix, False, 0)

    def generate_stream_with_suffix(self, req, prompt_suffix, abort_after=0):
        """Streams through a callback inside the engine; it fails the generation once it has seen
        `abort_after` tokens (0 = never).  stream_count() tells how many tokens it was handed."""
        return self._run(req, prompt_suffix, True, abort_after)

    def batch_device_ms(self):
        """Device time (HIP events) summed over the steps of the last request whose samples advanced together."""
        return self._L.rs_session_batch_device_ms(self._s)

    def bytes_per_token(self, kv_len):
        """Bytes one single-row decode step streams at the given live KV length (hipdec_bytes_per_token)."""
        return int(self._L.rs_session_bytes_per_token(self._s, kv_len))

    def stream_count(self):
        return int(self._L.rs_session_stream_count(self._s))


# ---------------------------------------------------------------- the server's session cache (bin/serve.rs:225-471)
class CacheGeneration:
    """serve.rs:241-246"""

    def __init__(self, batch, effective_prompt_tokens, prompt_truncated, cache_prefix_tokens):
        self.batch = batch
        self.effective_prompt_tokens = effective_prompt_tokens
        self.prompt_truncated = prompt_truncated
        self.cache_prefix_tokens = cache_prefix_tokens


class SessionCache:
    """LRU set of sessions keyed by prompt: exact hit, longest cached prefix + suffix prefill, or a new session."""

    def __init__(self, cfg, weights, softcap=0.0, max_entries=4, weight_dtype=0, kv_dtype=0, flags=0, ffn_activation=0):
        L = lib()
        self._L = L
        self.cfg = cfg
        rc = RsConfig.of(cfg, ffn_activation)
        keep, ptrs = [], (fp * (9 * cfg.nlayers))()
        for l, lw in enumerate(weights["layers"]):
            for k, nme in enumerate(_TENSORS):
                a = np.ascontiguousarray(lw[nme], np.float32)
                keep.append(a)
                ptrs[l * 9 + k] = a.ctypes.data_as(fp)
        gf = np.ascontiguousarray(weights["gamma_final"], np.float32)
        em = np.ascontiguousarray(weights["embed"], np.float32)
        self._w = C.c_void_p(L.rs_weights_from_arrays(C.byref(rc), ptrs, gf.ctypes.data_as(fp), em.ctypes.data_as(fp)))
        self._c = C.c_void_p(L.rs_session_cache_new(C.byref(rc), self._w, softcap, max_entries, int(weight_dtype),
                                                    int(kv_dtype), flags))

    def close(self):
        if getattr(self, "_c", None) and self._c.value:
            self._L.rs_session_cache_free(self._c)
            self._c = C.c_void_p()
        if getattr(self, "_w", None):
            self._L.rs_weights_free(self._w)
            self._w = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __len__(self):
        return int(self._L.rs_session_cache_len(self._c))

    def max_entries(self):
        return int(self._L.rs_session_cache_max_entries(self._c))

    def entry_prompt(self, i):
        n = self._L.rs_session_cache_entry_prompt(self._c, i, None, 0)
        out = np.empty(max(n, 1), np.uint32)
        self._L.rs_session_cache_entry_prompt(self._c, i, out.ctypes.data_as(u32p), out.size)
        return out[:n]

    def normalize_prompt_ids(self, prompt_ids):
        p = np.ascontiguousarray(prompt_ids, np.uint32)
        out = np.empty(max(p.size, 1), np.uint32)
        n = self._L.rs_session_cache_normalize(self._c, p.ctypes.data_as(u32p), p.size, out.ctypes.data_as(u32p), out.size)
        return out[:n]

    def find_exact(self, prompt_ids):
        p = np.ascontiguousarray(prompt_ids, np.uint32)
        return int(self._L.rs_session_cache_find(self._c, p.ctypes.data_as(u32p), p.size, 0))

    def find_longest_prefix(self, prompt_ids):
        p = np.ascontiguousarray(prompt_ids, np.uint32)
        return int(self._L.rs_session_cache_find(self._c, p.ctypes.data_as(u32p), p.size, 1))

    def insert(self, prompt_ids):
        p = np.ascontiguousarray(prompt_ids, np.uint32)
        err = C.create_string_buffer(512)
        idx = int(self._L.rs_session_cache_insert(self._c, p.ctypes.data_as(u32p), p.size, err, 512))
        if idx < 0:
            raise SessionError(err.value.decode())
        return idx

    def generate(self, prompt_ids, req, stream=False, abort_after=0):
        p = np.ascontiguousarray(prompt_ids, np.uint32)
        info, cinfo = RsBatchInfo(), (C.c_uint64 * 3)()
        err = C.create_string_buffer(512)
        rc = self._L.rs_session_cache_generate(self._c, p.ctypes.data_as(u32p), p.size, C.byref(req._c()), int(stream),
                                               abort_after, C.byref(info), cinfo, err, 512)
        if rc:
            raise SessionError(err.value.decode())
        results = []
        for i in range(info.n_results):
            arrs = []
            for which in (0, 1):
                n = self._L.rs_session_cache_result_len(self._c, i, which)
                a = np.empty(max(n, 1), np.uint32)
                self._L.rs_session_cache_result_copy(self._c, i, which, a.ctypes.data_as(u32p))
                arrs.append(a[:n])
            results.append(SampleResult(self._L.rs_session_cache_result_seed(self._c, i), arrs[1], arrs[0], 0.0))
        return CacheGeneration(GenerationBatch(info, results), int(cinfo[0]), bool(cinfo[1]), int(cinfo[2]))


# ---------------------------------------------------------------- RSTK checkpoints (crates/engine/src/checkpoint.rs)
class CheckpointError(ValueError):
    pass


_TENSORS = ("wq", "wk", "wv", "wo", "w1", "w3", "w2", "gamma1", "gamma2")


def _take_checkpoint(L, handle, rc, step):
    from .hipdec import Config
    cfg = Config.make(dim=rc.dim, hidden=rc.hidden, heads=rc.heads, hd=rc.hd, seq=rc.seq, nlayers=rc.nlayers,
                      vocab=rc.vocab, kv_heads=rc.kv_heads)

    def tensor(layer, which):
        p, n = fp(), C.c_uint64()
        if L.rs_weights_tensor(handle, layer, which, C.byref(p), C.byref(n)):
            raise CheckpointError("no such tensor")
        return np.ctypeslib.as_array(p, shape=(n.value,)).copy()

    try:
        weights = {"embed": tensor(-1, 0), "gamma_final": tensor(-1, 1),
                   "layers": [{nme: tensor(l, k) for k, nme in enumerate(_TENSORS)} for l in range(cfg.nlayers)]}
    finally:
        L.rs_weights_free(handle)
    return cfg, weights, int(step.value), int(rc.ffn_activation)


def parse_checkpoint(data):
    """checkpoint.rs:30-166 on a bytes object -> (cfg, weights dict, step, ffn_activation code)."""
    L = lib()
    rc, step, err = RsConfig(), C.c_uint32(), C.create_string_buffer(256)
    h = L.rs_checkpoint_parse(bytes(data), len(data), C.byref(rc), C.byref(step), err, 256)
    if not h:
        raise CheckpointError(err.value.decode())
    return _take_checkpoint(L, C.c_void_p(h), rc, step)


def load_checkpoint(path):
    """checkpoint.rs:25-28 -> (cfg, weights dict, step, ffn_activation code)."""
    L = lib()
    rc, step, err = RsConfig(), C.c_uint32(), C.create_string_buffer(512)
    h = L.rs_checkpoint_load(str(path).encode(), C.byref(rc), C.byref(step), err, 512)
    if not h:
        raise CheckpointError(err.value.decode())
    return _take_checkpoint(L, C.c_void_p(h), rc, step)


def write_checkpoint(path, cfg, weights, step=0, ffn_activation=0):
    """The version-2 file crates/engine/src/bin/train.rs:609-647 writes."""
    L = lib()
    rc = RsConfig.of(cfg, ffn_activation)
    keep, ptrs = [], (fp * (9 * cfg.nlayers))()
    for l, lw in enumerate(weights["layers"]):
        for k, nme in enumerate(_TENSORS):
            a = np.ascontiguousarray(lw[nme], np.float32)
            keep.append(a)
            ptrs[l * 9 + k] = a.ctypes.data_as(fp)
    gf = np.ascontiguousarray(weights["gamma_final"], np.float32)
    em = np.ascontiguousarray(weights["embed"], np.float32)
    h = C.c_void_p(L.rs_weights_from_arrays(C.byref(rc), ptrs, gf.ctypes.data_as(fp), em.ctypes.data_as(fp)))
    err = C.create_string_buffer(512)
    try:
        if L.rs_checkpoint_write(str(path).encode(), C.byref(rc), h, step, err, 512):
            raise CheckpointError(err.value.decode())
    finally:
        L.rs_weights_free(h)


def parse_packed_checkpoint(data):
    """Header and size check of a converted checkpoint (the weights as the decode library stores them for one
    weight format) -> (RsConfig fields as a dict, step, weight format code)."""
    L = lib()
    rc, step, dtype, err = RsConfig(), C.c_uint32(), C.c_uint32(), C.create_string_buffer(512)
    if L.rs_packed_checkpoint_parse(bytes(data), len(data), C.byref(rc), C.byref(step), C.byref(dtype), err, 512):
        raise CheckpointError(err.value.decode())
    return {k: int(getattr(rc, k)) for k, _ in RsConfig._fields_}, step.value, dtype.value


# ---------------------------------------------------------------- JSONL session protocol (bin/generate.rs:39-144)
class JsonlRequestError(ValueError):
    pass


def parse_jsonl_request(line, defaults=None):
    """One request line -> (GenerationRequest with the defaults filled in, appended prompt ids)."""
    L = lib()
    d = (defaults or GenerationRequest())._c()
    out, n, err = RsRequest(), C.c_uint64(), C.create_string_buffer(512)
    buf = np.zeros(4096, np.uint32)
    if L.rs_jsonl_parse(line.encode(), C.byref(d), C.byref(out), buf.ctypes.data_as(u32p), buf.size, C.byref(n), err, 512):
        raise JsonlRequestError(err.value.decode())
    req = GenerationRequest(DecodeBackendRequest(out.backend), out.steps, out.temperature, out.top_k, out.samples, out.seed)
    return req, buf[:n.value].copy()


# ---------------------------------------------------------------- HTTP front end (bin/serve.rs), the parts that need no model
class HttpRequestError(ValueError):
    """A request the server answers with status 400; `invalid_json` tells a body that does not parse from one
    that parses and is refused by validation."""

    def __init__(self, message, invalid_json=False):
        super().__init__(message)
        self.invalid_json = invalid_json


def http_parse_request(fd, max_body=64 << 20):
    """Reads one HTTP request from a connected socket -> (method, path, body bytes)."""
    L = lib()
    method, path, err = C.create_string_buffer(64), C.create_string_buffer(4096), C.create_string_buffer(512)
    cap = 1 << 20
    body, n = C.create_string_buffer(cap), C.c_uint64()
    if L.rs_http_parse_request(fd, max_body, method, 64, path, 4096, body, cap, C.byref(n), err, 512):
        raise HttpRequestError(err.value.decode())
    return method.value.decode(), path.value.decode(), body.raw[:min(n.value, cap)]


def http_prepare(body, chat=False, model_name="rustane", vocab=8192, default_backend=DecodeBackendRequest.AUTO):
    """The body of a (chat) completion request -> (prompt ids, GenerationRequest, stream flag), as the server
    derives them before generating (bin/serve.rs:635-725)."""
    L = lib()
    out, n, stream, err = RsRequest(), C.c_uint64(), C.c_int(), C.create_string_buffer(512)
    buf = np.zeros(4096, np.uint32)
    if isinstance(body, str):
        body = body.encode()
    rc = L.rs_http_prepare(body, int(chat), model_name.encode(), vocab, int(default_backend), C.byref(out), C.byref(stream),
                           buf.ctypes.data_as(C.POINTER(C.c_uint32)), buf.size, C.byref(n), err, 512)
    if rc:
        raise HttpRequestError(err.value.decode(), invalid_json=rc == 2)
    req = GenerationRequest(DecodeBackendRequest(out.backend), out.steps, out.temperature, out.top_k, out.samples, out.seed)
    return buf[:n.value].copy(), req, bool(stream.value)


def http_render_chat_prompt(body):
    """The flattened prompt text of a chat request's messages (bin/serve.rs:616-633)."""
    L = lib()
    out, err = C.create_string_buffer(1 << 16), C.create_string_buffer(512)
    if isinstance(body, str):
        body = body.encode()
    if L.rs_http_render_chat_prompt(body, out, 1 << 16, err, 512):
        raise HttpRequestError(err.value.decode(), invalid_json=True)
    return out.value.decode()
