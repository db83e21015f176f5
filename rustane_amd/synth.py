"""Synthetic weights and prompts for the benchmark configurations (ctypes view of csrc/engine/synth.cc)."""
import ctypes as C
import os

import numpy as np

from .hipdec import Config

_ENGINE = None
_ENGINE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "librustane_engine.so")


def load_engine():
    global _ENGINE
    if _ENGINE is None:
        if not os.path.exists(_ENGINE_PATH):
            raise RuntimeError("%s not found: build it with __graft_entry__.build()" % _ENGINE_PATH)
        lib = C.CDLL(_ENGINE_PATH)
        lib.rs_synth_normal.restype = None
        lib.rs_synth_normal.argtypes = [C.c_uint64, C.c_uint64, C.c_size_t, C.c_float, C.c_int, C.POINTER(C.c_float)]
        lib.rs_synth_prompt.restype = None
        lib.rs_synth_prompt.argtypes = [C.c_uint64, C.c_uint32, C.c_size_t, C.POINTER(C.c_uint32)]
        _ENGINE = lib
    return _ENGINE


def synth_normal(seed, tensor_id, n, std=0.02, round_bf16=False):
    out = np.empty(n, np.float32)
    load_engine().rs_synth_normal(seed, tensor_id, n, std, int(round_bf16), out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def layer_tensor_id(layer, k):
    return 16 * (layer + 1) + k


LAYER_TENSORS = ("wq", "wk", "wv", "wo", "w1", "w3", "w2")


def make_weights(cfg: Config, seed=1234, std=0.02, round_bf16=False):
    """Every matrix N(0, std) (including wo and w2, which the reference's own random init leaves
    at zero, crates/engine/src/layer.rs:706-709), all norm gains 1."""
    D, Q, KV, H, V = cfg.dim, cfg.q_dim, cfg.kv_dim, cfg.hidden, cfg.vocab
    sizes = dict(wq=D * Q, wk=D * KV, wv=D * KV, wo=Q * D, w1=D * H, w3=D * H, w2=D * H)
    layers = []
    for l in range(cfg.nlayers):
        lw = {name: synth_normal(seed, layer_tensor_id(l, k), sizes[name], std, round_bf16)
              for k, name in enumerate(LAYER_TENSORS)}
        lw["gamma1"] = np.ones(D, np.float32)
        lw["gamma2"] = np.ones(D, np.float32)
        layers.append(lw)
    return {"embed": synth_normal(seed, 0, V * D, std, round_bf16), "gamma_final": np.ones(D, np.float32),
            "layers": layers}


def make_prompt(seed, vocab, n):
    out = np.empty(n, np.uint32)
    load_engine().rs_synth_prompt(seed, vocab, n, out.ctypes.data_as(C.POINTER(C.c_uint32)))
    return out


# The five benchmark configurations.
def config_c1():
    return Config.make(dim=512, hidden=1536, heads=8, hd=64, seq=512, nlayers=8, vocab=8192)


def config_600m():
    return Config.make(dim=1536, hidden=4096, heads=12, hd=128, seq=2048, nlayers=24, vocab=32768)


def config_5b():
    return Config.make(dim=4096, hidden=11008, heads=32, hd=128, seq=4096, nlayers=32, vocab=32768)
