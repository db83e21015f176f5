"""hipdec_sample_fullvocab_noalloc -- the full-vocabulary draw for callers that cannot allocate.

Same draw as hipdec_debug_sample_fullvocab (engine/src/inference.rs:851-921 on the device), but on
device buffers, on the caller's stream, with the kernels' run state in an array the library holds on
the GPU.  Checked token for token and RNG state for RNG state against that entry point (and so,
through tests/test_device_sampling.py, against the oracle's two draws), on consecutive calls that
share the array -- the second with a smaller vocabulary -- and on the argument errors.
The HIP runtime (through ctypes) only supplies the device buffers and the stream."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O
from rustane_amd import hipdec


class Hip:
    """The few HIP runtime calls the test needs for device buffers (the runtime libhipdecode.so links)."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipStreamDestroy.argtypes = [C.c_void_p]
        self.rt.hipStreamSynchronize.argtypes = [C.c_void_p]
        self.rt.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        self.rt.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        self.rt.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        self.rt.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipGraphExecDestroy.argtypes = [C.c_void_p]
        self.rt.hipGraphDestroy.argtypes = [C.c_void_p]
        self.bufs = []

    def ok(self, rc):
        assert rc == 0, "HIP runtime call failed with %d" % rc

    def put(self, a):
        a = np.ascontiguousarray(a)
        p = C.c_void_p()
        self.ok(self.rt.hipMalloc(C.byref(p), max(a.nbytes, 16)))
        self.bufs.append(p)
        self.ok(self.rt.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), a.nbytes, 1))      # host -> device
        return p.value

    def get(self, ptr, dtype, n):
        out = np.empty(n, dtype)
        self.ok(self.rt.hipMemcpy(out.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), out.nbytes, 2))   # device -> host
        return out

    def sync(self):
        self.ok(self.rt.hipDeviceSynchronize())

    def stream(self):
        s = C.c_void_p()
        self.ok(self.rt.hipStreamCreate(C.byref(s)))
        return s

    def free_all(self):
        self.sync()
        for p in self.bufs:
            self.rt.hipFree(p)
        self.bufs = []


def _draw_pair(hip, logits, T, seed, softcap=0.0, stream=None):
    """(no-alloc result, existing entry point's result) for one draw."""
    V = logits.size
    inv_t = float(np.float32(1.0) / np.float32(T))
    with np.errstate(invalid="ignore"):
        mx, sm = O.block_stats(logits, inv_t, softcap)
    want = hipdec.debug_sample_fullvocab(logits, mx, sm, T, seed, softcap=softcap)
    d_lg, d_mx, d_sm = hip.put(logits), hip.put(mx), hip.put(sm)
    d_rng = hip.put(np.array([seed], np.uint64))
    d_tok = hip.put(np.array([0xFFFFFFFF], np.uint32))
    hip.sync()
    hipdec.sample_fullvocab_noalloc(d_lg, V, d_mx, d_sm, T, d_rng, d_tok, softcap=softcap, stream=stream)
    hip.sync()
    got = (int(hip.get(d_tok, np.uint32, 1)[0]), int(hip.get(d_rng, np.uint64, 1)[0]))
    hip.free_all()
    return got, want


@pytest.mark.gpu
def test_noalloc_draw_equals_the_allocating_entry_point_on_consecutive_calls():
    hip = Hip()
    rng = np.random.default_rng(5)
    # two calls in a row share the library's run-state array; the second has the smaller input
    big = (rng.standard_normal(32768) * 3.0).astype(np.float32)
    small = (rng.standard_normal(1000) * 3.0).astype(np.float32)
    got, want = _draw_pair(hip, big, 1.0, 77)
    assert got == want, (got, want)
    got, want = _draw_pair(hip, small, 0.7, 78)
    assert got == want, (got, want)
    # more draws: a softcap, a vocabulary that ends inside a block, the maximum size, dead blocks,
    # a stream that is not the default one
    side = hip.stream()
    seed = 100
    for V, T, cap in ((257, 2.0, 0.0), (8192, 0.3, 5.0), (262144, 1.0, 0.0), (320, 1.0, 0.0), (256, 0.9, 0.0)):
        lg = (rng.standard_normal(V) * 4.0).astype(np.float32)
        if V == 320:
            lg[:256] = -np.inf
        for rep in range(3):
            seed += 1
            got, want = _draw_pair(hip, lg, T, seed, softcap=cap, stream=side if rep == 2 else None)
            assert got == want, (V, T, cap, rep, got, want)
    hip.ok(hip.rt.hipStreamDestroy(side))


@pytest.mark.gpu
def test_noalloc_draw_recorded_into_a_graph_replays_like_the_eager_call():
    """The use the entry point is for: recorded under stream capture (kernel nodes only -- it clears its
    run state with a kernel, not a memset) and replayed, with the caller's own eager copies and waits
    between the replays; every replay against the allocating entry point's draw."""
    hip = Hip()
    rng = np.random.default_rng(9)
    V, T = 5000, 0.9
    logits = (rng.standard_normal(V) * 3.0).astype(np.float32)
    inv_t = float(np.float32(1.0) / np.float32(T))
    mx, sm = O.block_stats(logits, inv_t, 0.0)
    d_lg, d_mx, d_sm = hip.put(logits), hip.put(mx), hip.put(sm)
    d_rng = hip.put(np.array([1], np.uint64))
    d_tok = hip.put(np.array([0xFFFFFFFF], np.uint32))
    s = hip.stream()
    # the first call on a device looks the scratch array up, which is not a capturable operation (creating a
    # model does the same): one eager call, then the capture
    hipdec.sample_fullvocab_noalloc(d_lg, V, d_mx, d_sm, T, d_rng, d_tok, stream=s)
    hip.ok(hip.rt.hipStreamSynchronize(s))
    hip.ok(hip.rt.hipStreamBeginCapture(s, 1))                       # thread-local capture
    hipdec.sample_fullvocab_noalloc(d_lg, V, d_mx, d_sm, T, d_rng, d_tok, stream=s)
    graph, gexec = C.c_void_p(), C.c_void_p()
    hip.ok(hip.rt.hipStreamEndCapture(s, C.byref(graph)))
    hip.ok(hip.rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0))
    for seed in (41, 42, 43):
        want = hipdec.debug_sample_fullvocab(logits, mx, sm, T, seed)
        one = np.array([seed], np.uint64)
        hip.ok(hip.rt.hipMemcpy(C.c_void_p(d_rng), one.ctypes.data_as(C.c_void_p), 8, 1))
        none = np.array([0xFFFFFFFF], np.uint32)
        hip.ok(hip.rt.hipMemcpy(C.c_void_p(d_tok), none.ctypes.data_as(C.c_void_p), 4, 1))
        hip.ok(hip.rt.hipGraphLaunch(gexec, s))
        hip.ok(hip.rt.hipStreamSynchronize(s))
        got = (int(hip.get(d_tok, np.uint32, 1)[0]), int(hip.get(d_rng, np.uint64, 1)[0]))
        assert got == want, (seed, got, want)
    hip.ok(hip.rt.hipGraphExecDestroy(gexec))
    hip.ok(hip.rt.hipGraphDestroy(graph))
    hip.ok(hip.rt.hipStreamDestroy(s))
    hip.free_all()


@pytest.mark.gpu
def test_noalloc_draw_rejects_bad_arguments_without_touching_the_outputs():
    hip = Hip()
    p = hip.put(np.zeros(2048, np.float32))
    rng = hip.put(np.zeros(1, np.uint64))
    tok = hip.put(np.array([7], np.uint32))
    for args in ((p, 262145, p, p, 1.0, rng, tok),      # beyond the 1024-block maximum
                 (p, 0, p, p, 1.0, rng, tok),
                 (p, 1000, p, p, 0.0, rng, tok),        # temperature must be positive
                 (None, 1000, p, p, 1.0, rng, tok),
                 (p, 1000, p, p, 1.0, None, tok)):
        with pytest.raises(hipdec.HipDecodeError) as ei:
            hipdec.sample_fullvocab_noalloc(*args)
        assert ei.value.status == hipdec.ERR_ARG
    with pytest.raises(hipdec.HipDecodeError, match="262144"):
        hipdec.sample_fullvocab_noalloc(p, 1 << 20, p, p, 1.0, rng, tok)
    hip.sync()
    assert int(hip.get(tok, np.uint32, 1)[0]) == 7 and int(hip.get(rng, np.uint64, 1)[0]) == 0
    hip.free_all()
