"""RSTK checkpoint reader/writer of the host engine against the format the reference defines
(crates/engine/src/checkpoint.rs:1-242, writer crates/engine/src/bin/train.rs:609-647).  The files
under test are assembled here with numpy straight from that description, the way the reference's
own test assembles them (checkpoint.rs:262-313), so the reader is not checked against its own writer
alone; every rejection the reference's parser has is provoked with its message."""
import struct

import numpy as np
import pytest

from rustane_amd import engine, synth
from rustane_amd.hipdec import Config

NAMES = ("wq", "wk", "wv", "wo", "w1", "w3", "w2", "gamma1", "gamma2")


def cfg_small(hidden=640):
    # the shape of the reference's own parser test (checkpoint.rs:264-277)
    return Config.make(dim=256, hidden=hidden, heads=2, hd=128, seq=64, nlayers=2, vocab=32)


def file_bytes(cfg, w, version=2, step=123, act=0, magic=b"RSTK"):
    head = magic + struct.pack("<I", version) + struct.pack("<5I", step, cfg.dim, cfg.nlayers, cfg.vocab, cfg.seq)
    if version >= 2:
        head += struct.pack("<I", act)
    parts = [head, np.asarray(w["embed"], "<f4").tobytes(), np.asarray(w["gamma_final"], "<f4").tobytes()]
    for lw in w["layers"]:
        parts += [np.asarray(lw[n], "<f4").tobytes() for n in NAMES]
    return b"".join(parts)


def assert_same_weights(a, b):
    np.testing.assert_array_equal(a["embed"], b["embed"])
    np.testing.assert_array_equal(a["gamma_final"], b["gamma_final"])
    assert len(a["layers"]) == len(b["layers"])
    for la, lb in zip(a["layers"], b["layers"]):
        for n in NAMES:
            np.testing.assert_array_equal(la[n], lb[n])


@pytest.mark.parametrize("hidden,act", [(640, 0), (384, 1)])
def test_parses_checkpoint_and_infers_hidden(hidden, act):
    cfg = cfg_small(hidden)
    w = synth.make_weights(cfg, seed=3, std=0.05)
    got_cfg, got_w, step, got_act = engine.parse_checkpoint(file_bytes(cfg, w, act=act))
    assert step == 123 and got_act == act
    for f in ("dim", "hidden", "heads", "kv_heads", "hd", "seq", "nlayers", "vocab", "q_dim", "kv_dim"):
        assert getattr(got_cfg, f) == getattr(cfg, f), f
    assert_same_weights(got_w, w)


def test_version_1_has_no_activation_field():
    cfg = cfg_small()
    w = synth.make_weights(cfg, seed=4, std=0.05)
    got_cfg, got_w, step, act = engine.parse_checkpoint(file_bytes(cfg, w, version=1, step=7))
    assert (step, act, got_cfg.hidden) == (7, 0, 640)
    assert_same_weights(got_w, w)


def test_rejections_carry_the_reference_messages():
    cfg = cfg_small()
    w = synth.make_weights(cfg, seed=5, std=0.05)
    good = file_bytes(cfg, w)

    def msg(data):
        with pytest.raises(engine.CheckpointError) as e:
            engine.parse_checkpoint(data)
        return str(e.value)

    assert msg(good[:20]) == "checkpoint too small for header"
    assert msg(file_bytes(cfg, w, magic=b"RSTX")) == "invalid checkpoint magic"
    assert msg(file_bytes(cfg, w, version=3)) == "unsupported checkpoint version 3"
    assert msg(file_bytes(cfg, w, version=0)) == "unsupported checkpoint version 0"
    assert msg(b"RSTK" + struct.pack("<6I", 2, 0, 256, 2, 32, 64)) == "checkpoint too small for v2 header"
    assert msg(file_bytes(cfg, w, act=2)) == "unsupported checkpoint activation code 2"
    zero = bytearray(good); zero[12:16] = struct.pack("<I", 0)
    assert msg(bytes(zero)) == "checkpoint config contains zero dimension"
    odd = bytearray(good); odd[12:16] = struct.pack("<I", 200)
    assert msg(bytes(odd)) == "checkpoint dim 200 is not divisible by 128"
    assert msg(good + b"\0\0") == "checkpoint payload is not aligned to f32 values"
    assert msg(good[:32 + 4 * 100]) == "checkpoint payload too small for fixed-size tensors"
    assert msg(good + b"\0" * 4) == "checkpoint payload does not imply an integer hidden size"


def test_writer_emits_the_documented_layout_and_round_trips(tmp_path):
    cfg = cfg_small()
    w = synth.make_weights(cfg, seed=6, std=0.05)
    path = tmp_path / "ckpt_000042.bin"
    engine.write_checkpoint(path, cfg, w, step=42, ffn_activation=1)
    assert path.read_bytes() == file_bytes(cfg, w, step=42, act=1)
    got_cfg, got_w, step, act = engine.load_checkpoint(path)
    assert (step, act, got_cfg.hidden) == (42, 1, 640)
    assert_same_weights(got_w, w)
    with pytest.raises(engine.CheckpointError):
        engine.load_checkpoint(tmp_path / "missing.bin")


def test_models_the_header_cannot_describe_round_trip_through_the_shape_file(tmp_path):
    """The header has no place for hd, kv_heads or hidden (checkpoint.rs:83-112 assumes hd 128, MHA and
    infers hidden): such a model keeps the reference's file layout and gets PATH.shape beside it."""
    gqa = Config.make(dim=192, hidden=320, heads=3, hd=64, seq=64, nlayers=2, vocab=48, kv_heads=1)   # the tiny workload's kind
    w = synth.make_weights(gqa, seed=1, std=0.05)
    path = tmp_path / "tiny.bin"
    engine.write_checkpoint(path, gqa, w, step=9, ffn_activation=1)
    assert (tmp_path / "tiny.bin.shape").read_text() == "heads=3 kv_heads=1 hd=64 hidden=320\n"
    assert path.read_bytes() == file_bytes(gqa, w, step=9, act=1)            # the main file is the documented layout
    cfg2, w2, step, act = engine.load_checkpoint(path)
    assert (step, act) == (9, 1)
    assert (cfg2.dim, cfg2.hidden, cfg2.heads, cfg2.kv_heads, cfg2.hd, cfg2.q_dim, cfg2.kv_dim) == (192, 320, 3, 1, 64, 192, 64)
    assert_same_weights(w2, w)
    # without the side file the main file is read as the reference reads it: rejected here (dim % 128)
    with pytest.raises(engine.CheckpointError, match="checkpoint dim 192 is not divisible by 128"):
        engine.parse_checkpoint(path.read_bytes())
    # a side file that does not fit the payload, or does not parse
    (tmp_path / "tiny.bin.shape").write_text("heads=3 kv_heads=1 hd=64 hidden=352\n")
    with pytest.raises(engine.CheckpointError, match="does not match the shape file"):
        engine.load_checkpoint(path)
    (tmp_path / "tiny.bin.shape").write_text("heads=3 kv_heads=2 hd=64 hidden=320\n")
    with pytest.raises(engine.CheckpointError, match="no valid model"):
        engine.load_checkpoint(path)
    (tmp_path / "tiny.bin.shape").write_text("heads=3 hd=64\n")
    with pytest.raises(engine.CheckpointError, match="must read: heads=H kv_heads=K hd=E hidden=F"):
        engine.load_checkpoint(path)
    # a model the header describes leaves no side file behind, and removes a stale one
    cfg = cfg_small()
    engine.write_checkpoint(path, cfg, synth.make_weights(cfg, seed=6, std=0.05), step=1)
    assert not (tmp_path / "tiny.bin.shape").exists()
    assert engine.load_checkpoint(path)[0].hd == 128


@pytest.mark.gpu
def test_session_from_checkpoint_equals_session_from_arrays(tmp_path):
    cfg = cfg_small()
    w = synth.make_weights(cfg, seed=8, std=0.08, round_bf16=True)
    path = tmp_path / "ckpt.bin"
    engine.write_checkpoint(path, cfg, w, step=1)
    cfg2, w2, _, act = engine.load_checkpoint(path)
    prompt = synth.make_prompt(3, cfg.vocab, 9)
    req = engine.GenerationRequest(decode_backend=engine.DecodeBackendRequest.HIP, steps=12, temperature=0.0)
    a = engine.InferenceSession(cfg, w, prompt, weight_dtype=1, kv_dtype=0).generate(req)
    b = engine.InferenceSession(cfg2, w2, prompt, weight_dtype=1, kv_dtype=0, ffn_activation=act).generate(req)
    np.testing.assert_array_equal(a.results[0].sampled, b.results[0].sampled)


# ---------------------------------------------------------------- converted checkpoints (this build's "RSTQ" file)
def _packed_bytes(cfg, dtype, step=7, act=0, version=1, extra=0):
    """A converted checkpoint of the right size for (cfg, weight format), built from the format description."""
    import ctypes as C
    from rustane_amd import hipdec

    class Sizes(C.Structure):
        _fields_ = [(n, C.c_uint64) for n in ("wqkv", "wo", "w13", "w2", "s_qkv", "s_wo", "s_w13", "s_w2", "gamma", "embed")]

    lib = hipdec.load_library()
    z = Sizes()
    rc = lib.hipdec_packed_sizes_of(C.byref(cfg), dtype, C.byref(z))
    if rc:
        return None, rc
    per_layer = z.wqkv + z.s_qkv + z.wo + z.s_wo + z.w13 + z.s_w13 + z.w2 + z.s_w2 + 2 * z.gamma
    head = b"RSTQ" + np.array([version, step, dtype, act, cfg.dim, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.hd, cfg.seq,
                               cfg.nlayers, cfg.vocab], np.uint32).tobytes()
    return head + bytes(z.gamma + z.embed + cfg.nlayers * per_layer + extra), 0


def test_converted_checkpoint_header_and_sizes():
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=64, nlayers=3, vocab=320)
    sizes = {}
    for dtype in (0, 1, 2, 3):
        data, rc = _packed_bytes(cfg, dtype, step=41, act=1 if dtype == 2 else 0)
        assert rc == 0
        got, step, dt = engine.parse_packed_checkpoint(data)
        assert (step, dt) == (41, dtype) and got["ffn_activation"] == (1 if dtype == 2 else 0)
        assert [got[k] for k in ("dim", "hidden", "heads", "kv_heads", "hd", "seq", "nlayers", "vocab")] == \
               [256, 640, 2, 2, 128, 64, 3, 320]
        sizes[dtype] = len(data)
    # fp32 : bf16 : e4m3 : 4-bit matrices are 4 : 2 : 1 : 0.5 bytes per weight (+ scales, norms and the bf16 embedding)
    assert sizes[0] > sizes[1] > sizes[2] > sizes[3]
    lin = 3 * (4 * 256 * 256 + 3 * 256 * 640)
    assert sizes[1] - sizes[2] == lin - 3 * 4 * (768 + 256 + 1280 + 256)          # one byte less per weight, one fp32 scale per row more
    assert sizes[2] - sizes[3] == lin // 2 + 3 * 4 * (768 + 256 + 1280 + 256) - 3 * 2 * (768 * 2 + 256 * 2 + 1280 * 2 + 256 * 5)


def test_converted_checkpoint_rejections():
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=64, nlayers=2, vocab=320)

    def msg(data):
        with pytest.raises(engine.CheckpointError) as e:
            engine.parse_packed_checkpoint(data)
        return str(e.value)

    good, _ = _packed_bytes(cfg, 1)
    assert msg(good[:40]) == "converted checkpoint too small for header"
    assert msg(b"RSTK" + good[4:]) == "bad converted checkpoint magic"
    assert msg(_packed_bytes(cfg, 1, version=2)[0]) == "unsupported converted checkpoint version 2"
    bad = bytearray(good); bad[12:16] = np.uint32(9).tobytes()
    assert msg(bytes(bad)) == "unknown weight format 9 in converted checkpoint"
    bad = bytearray(good); bad[16:20] = np.uint32(5).tobytes()
    assert msg(bytes(bad)) == "unknown ffn activation 5 in converted checkpoint"
    bad = bytearray(good); bad[20:24] = np.uint32(0).tobytes()
    assert msg(bytes(bad)) == "converted checkpoint header describes no model"
    assert "does not match its header" in msg(good + b"\0")
    assert "does not match its header" in msg(good[:-4])
    # a shape the weight format cannot hold (4-bit groups of 128 along every reduction axis)
    odd = bytearray(good); odd[12:16] = np.uint32(3).tobytes(); odd[24:28] = np.uint32(704).tobytes()
    assert "multiples of the weight load width" in msg(bytes(odd))


def _generate(*args):
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    return subprocess.run([os.path.join(root, "rustane_amd", "lib", "generate")] + [str(a) for a in args],
                          capture_output=True, text=True, timeout=120)


def _ids(stdout, key="generated_ids="):
    return [ln[len(key):] for ln in stdout.splitlines() if ln.startswith(key)]


@pytest.mark.gpu
@pytest.mark.parametrize("wdt,code", [("f32", 0), ("bf16", 1), ("fp8", 2), ("int4", 3)])
def test_converted_checkpoint_generates_what_the_fp32_file_generates(tmp_path, wdt, code):
    # offline conversion: generate --convert-to writes the weights as the device stores them for one format;
    # a model created from that file (plain copies, no conversion) must give the very tokens of a model
    # converted from the fp32 file at creation -- greedy and sampled
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=3, vocab=320)
    w = synth.make_weights(cfg, seed=12, std=0.08, round_bf16=False)
    src, dst = tmp_path / "ckpt_000009.bin", tmp_path / "ckpt_000009.rstq"
    engine.write_checkpoint(src, cfg, w, step=9)
    p = _generate("--checkpoint", src, "--weight-dtype", wdt, "--convert-to", dst)
    assert p.returncode == 0, p.stderr
    assert p.stdout.splitlines()[-1] == "converted_checkpoint=%s weight_dtype=%s step=9" % (dst, wdt)
    data = dst.read_bytes()
    got, step, dt = engine.parse_packed_checkpoint(data)
    assert (step, dt, got["dim"], got["hidden"], got["nlayers"], got["vocab"]) == (9, code, 256, 640, 3, 320)
    assert len(data) == len(_packed_bytes(cfg, code)[0])
    common = ["--prompt-ids", "3,1,4,1,5,9,2,6,5,3,5", "--decode-backend", "hip", "--kv-dtype", "bf16"]
    for extra in (["--steps", "12"], ["--steps", "10", "--temperature", "0.8", "--top-k", "6", "--samples", "3", "--seed", "5"]):
        a = _generate("--checkpoint", src, "--weight-dtype", wdt, *common, *extra)
        b = _generate("--checkpoint", dst, *common, *extra)                    # (the file names its weight format)
        assert a.returncode == 0 and b.returncode == 0, a.stderr + b.stderr
        key = "generated_ids=" if "--samples" not in extra else "sample"
        ia = [ln for ln in a.stdout.splitlines() if ln.startswith(key) and "_ids=" in ln]
        ib = [ln for ln in b.stdout.splitlines() if ln.startswith(key) and "_ids=" in ln]
        assert ia and ia == ib
        assert "loaded checkpoint: step=9 model=3L 256D 640H 320V seq=96" in b.stdout
    # the format is the file's: naming another one is refused, and a converted file is not converted again
    bad = _generate("--checkpoint", dst, "--weight-dtype", "bf16" if wdt != "bf16" else "int4", *common)
    assert bad.returncode == 2 and "does not match the format this converted checkpoint holds" in bad.stderr
    again = _generate("--checkpoint", dst, "--convert-to", tmp_path / "x.rstq")
    assert again.returncode == 2 and "converted already" in again.stderr
