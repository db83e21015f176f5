"""The HTTP front end of the server (crates/engine/src/bin/serve.rs:473-1281): request parsing, validation
and the routes that need no model on the CPU; on the GPU the `serve` binary is driven over a loopback
socket and its answers (JSON and server-sent events) are compared with direct session-cache calls."""
import http.client
import json
import os
import socket
import subprocess
import threading
import time

import pytest

from rustane_amd import engine, synth
from rustane_amd.hipdec import Config

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SERVE = os.path.join(ROOT, "rustane_amd", "lib", "serve")
AUTO, NAIVE, HIP = engine.DecodeBackendRequest.AUTO, engine.DecodeBackendRequest.NAIVE, engine.DecodeBackendRequest.HIP


# ---------------------------------------------------------------- reading a request off a socket (serve.rs:877-927)
def _parse(raw, **kw):
    a, b = socket.socketpair()

    def send():                                   # (a big request does not fit the socket buffer: send while the parser reads)
        try:
            a.sendall(raw)
            a.shutdown(socket.SHUT_WR)
        except OSError:
            pass

    t = threading.Thread(target=send)
    t.start()
    try:
        return engine.http_parse_request(b.fileno(), **kw)
    finally:
        b.close()
        t.join()
        a.close()


def test_request_line_headers_and_body():
    body = b'{"prompt_ids":[1,2,3]}'
    raw = b"POST /v1/completions HTTP/1.1\r\nHost: x\r\nCONTENT-length:  %d \r\nX-No-Colon\r\n\r\n%s" % (len(body), body)
    assert _parse(raw) == ("POST", "/v1/completions", body)
    # bare line feeds, no body, bytes after the declared length are not read
    assert _parse(b"GET /healthz HTTP/1.1\nAccept: */*\n\nextra") == ("GET", "/healthz", b"")
    big = b"x" * 300000                                     # a body that arrives in many reads
    assert _parse(b"POST /p HTTP/1.1\r\nContent-Length: 300000\r\n\r\n" + big) == ("POST", "/p", big)


def test_request_rejections():
    def msg(raw, **kw):
        with pytest.raises(engine.HttpRequestError) as e:
            _parse(raw, **kw)
        return str(e.value)

    assert msg(b"") == "empty request"
    assert msg(b"   \r\n\r\n") == "empty request"
    assert msg(b"GET\r\n\r\n") == "missing HTTP path"
    assert msg(b"POST /x HTTP/1.1\r\nContent-Length: abc\r\n\r\n") == "invalid content-length"
    assert msg(b"POST /x HTTP/1.1\r\nContent-Length: -1\r\n\r\n") == "invalid content-length"
    assert msg(b"POST /x HTTP/1.1\r\nContent-Length: 10\r\n\r\nshort").startswith("failed to read request body: ")
    assert msg(b"POST /x HTTP/1.1\r\nContent-Length: 100\r\n\r\n" + b"y" * 100, max_body=99) == "request body too large"
    assert msg(b"GET /" + b"a" * 70000 + b" HTTP/1.1\r\n\r\n").startswith("failed to read request line: ")


# ---------------------------------------------------------------- request bodies (serve.rs:30-57, :635-725)
def test_completion_fields_and_defaults():
    ids, req, stream = engine.http_prepare('{"prompt_ids":[5,6,7]}')
    assert ids.tolist() == [5, 6, 7] and not stream
    assert (req.decode_backend, req.steps, req.temperature, req.top_k, req.samples, req.seed) == (AUTO, 32, 0.0, 0, 1, 1)
    body = ' {"model":"m","prompt_ids":[1, 2],"max_tokens":7,"temperature":0.75,"top_k":9,"seed":18446744073709551615,' \
           '"n":3,"stream":true,"decode_backend":"naive","add_special_tokens":false,"user":{"x":[1,null,"y"]}} '
    ids, req, stream = engine.http_prepare(body, model_name="m", default_backend=HIP)
    assert ids.tolist() == [1, 2] and stream
    assert (req.decode_backend, req.steps, req.temperature, req.top_k, req.samples, req.seed) == (NAIVE, 7, 0.75, 9, 3, 2 ** 64 - 1)
    # Option<T>: null is "not given"; the server's default backend applies
    ids, req, stream = engine.http_prepare('{"prompt_ids":[4],"max_tokens":null,"n":null,"stream":null,"model":null,'
                                           '"decode_backend":null}', default_backend=HIP)
    assert (req.decode_backend, req.steps, req.samples, stream) == (HIP, 32, 1, False)


def test_completion_rejections():
    def msg(body, **kw):
        with pytest.raises(engine.HttpRequestError) as e:
            engine.http_prepare(body, **kw)
        return str(e.value), e.value.invalid_json

    for body in ("not json", '{"max_tokens":-1,"prompt_ids":[1]}', '{"n":1.5,"prompt_ids":[1]}', '{"prompt_ids":[1,4294967296]}',
                 '{"prompt_ids":[1]} x', '{"stream":"yes","prompt_ids":[1]}', '{"prompt_ids":{"a":1}}', '[1]'):
        m, invalid = msg(body)
        assert invalid and m.startswith("invalid JSON: "), body
    m, invalid = msg('{"x":' + "[" * 100000 + "]" * 100000 + ',"prompt_ids":[1]}')      # (skipping an unknown field recurses)
    assert invalid and "nested too deeply" in m
    ids, _, _ = engine.http_prepare('{"x":' + "[" * 100 + "]" * 100 + ',"prompt_ids":[1]}')
    assert ids.tolist() == [1]
    assert msg('{"model":"other","prompt_ids":[1]}') == ("requested model other does not match loaded model rustane", False)
    assert msg('{"prompt":"a","prompt_ids":[1]}')[0] == "pass either prompt or prompt_ids, not both"
    assert msg('{}')[0] == "one of prompt or prompt_ids is required"
    assert msg('{"prompt":"hello"}')[0].startswith("failed to encode prompt: ")          # no tokenizer in this build
    assert msg('{"prompt_ids":[]}')[0] == "prompt encoded to zero tokens"
    assert msg('{"prompt_ids":[3,8192]}')[0] == "prompt token id 8192 at position 1 exceeds model vocab 8192"
    assert msg('{"prompt_ids":[1],"n":0}')[0] == "n must be >= 1"
    assert msg('{"prompt_ids":[1],"decode_backend":"cuda"}')[0] == "decode_backend must be one of: auto, naive, hip; got cuda"
    assert msg('{"prompt_ids":[1],"decode_backend":"metal"}')[0].startswith("decode_backend metal is the Apple-GPU backend")
    # the model is checked before the prompt, the prompt before the generation fields (serve.rs:662-691)
    assert msg('{"model":"other","n":0}')[0].startswith("requested model")
    assert msg('{"n":0}')[0] == "one of prompt or prompt_ids is required"


def test_chat_requests():
    body = json.dumps({"messages": [{"role": "system", "content": "  Be terse \n"}, {"role": "user", "content": "Hello"},
                                    {"role": "tool", "content": "\tx"}]})
    assert engine.http_render_chat_prompt(body) == "Be terse\n\nHello\n\nx"      # serve.rs:1346-1358: every role alike
    ids, req, stream = engine.http_prepare(json.dumps({"messages": [{"role": "system", "content_ids": [9, 8]},
                                                                    {"role": "user", "content_ids": [7], "content": " "}],
                                                       "max_tokens": 3, "prompt_ids": [1]}), chat=True)
    assert ids.tolist() == [9, 8, 7] and req.steps == 3 and not stream          # (prompt_ids is no field of a chat request)

    def msg(body):
        with pytest.raises(engine.HttpRequestError) as e:
            engine.http_prepare(body, chat=True)
        return str(e.value), e.value.invalid_json

    assert msg('{"messages":[]}') == ("messages must contain at least one item", False)
    assert msg('{"max_tokens":3}') [1] and "messages" in msg('{"max_tokens":3}')[0]
    assert msg('{"messages":null}')[1]
    assert msg('{"messages":[{"content":"x"}]}')[1] and "role" in msg('{"messages":[{"content":"x"}]}')[0]
    assert msg('{"messages":[{"role":"user"}]}')[1]
    assert msg('{"messages":[{"role":"user","content":"hi"}]}')[0].startswith("failed to encode prompt: ")
    assert msg('{"messages":[{"role":"user","content_ids":[]}]}')[0] == "prompt encoded to zero tokens"


# ---------------------------------------------------------------- the binary
class Server:
    def __init__(self, args):
        self.proc = subprocess.Popen([SERVE, "--bind", "127.0.0.1:0"] + args, stderr=subprocess.PIPE, text=True)
        self.ready = self.proc.stderr.readline().strip()
        assert self.ready.startswith("rustane_serve_ready bind=127.0.0.1:"), self.ready + self.proc.stderr.read()
        self.port = int(self.ready.split()[1].rsplit(":", 1)[1])

    def request(self, method, path, body=None, raw=False):
        c = http.client.HTTPConnection("127.0.0.1", self.port, timeout=120)
        if body is not None and not isinstance(body, (bytes, str)):
            body = json.dumps(body)
        c.request(method, path, body=body)
        r = c.getresponse()
        data = r.read()
        c.close()
        return r.status, r.reason, dict(r.getheaders()), data if raw else json.loads(data)

    def events(self, path, body):
        """A streamed answer: (headers, the JSON of every data event, whether it ended with [DONE])."""
        status, _, headers, data = self.request("POST", path, body, raw=True)
        assert status == 200
        ev = [e[len("data: "):] for e in data.decode().split("\n\n") if e]
        assert all(e.startswith("data: ") for e in data.decode().split("\n\n") if e)
        return headers, [json.loads(e) for e in ev if e != "[DONE]"], ev[-1] == "[DONE]"

    def close(self):
        self.proc.terminate()
        try:
            self.proc.wait(timeout=10)
        except subprocess.TimeoutExpired:
            self.proc.kill()
        self.proc.stderr.close()


def _error(message):
    return {"error": {"message": message, "type": "invalid_request_error"}}


def test_routes_that_need_no_model():
    srv = Server(["--model", "custom:256,640,2,96,2,128,320", "--model-name", "tiny", "--max-cache-sessions", "5"])
    try:
        assert srv.ready == "rustane_serve_ready bind=127.0.0.1:%d model=tiny vocab=320 seq=96 cache_sessions=5" % srv.port
        status, reason, headers, body = srv.request("GET", "/healthz")
        assert (status, reason) == (200, "OK") and headers["Content-Type"] == "application/json" and headers["Connection"] == "close"
        assert body == {"ok": True, "model": "tiny", "vocab": 320, "seq": 96, "cache_entries": 0, "max_cache_sessions": 5}
        assert list(body) == ["ok", "model", "vocab", "seq", "cache_entries", "max_cache_sessions"]
        assert srv.request("GET", "/v1/models")[3] == {"object": "list", "data": [{"id": "tiny", "object": "model", "owned_by": "rustane"}]}
        assert srv.request("GET", "/nope")[::3] == (404, _error("unknown route"))
        assert srv.request("POST", "/v1/nope", {})[::3] == (404, _error("unknown route"))
        assert srv.request("DELETE", "/healthz")[:2] + srv.request("PUT", "/v1/completions", {})[3:] == \
               (405, "Method Not Allowed", _error("unsupported HTTP method"))
        status, _, _, body = srv.request("POST", "/v1/completions", "{broken")
        assert status == 400 and body["error"]["message"].startswith("invalid JSON: ")
        assert srv.request("POST", "/v1/completions", {"prompt_ids": [1, 320]})[::3] == \
               (400, _error("prompt token id 320 at position 1 exceeds model vocab 320"))
        assert srv.request("POST", "/v1/completions", {"prompt_ids": [1], "stream": True, "n": 2})[::3] == \
               (400, _error("stream=true only supports n=1"))
        assert srv.request("POST", "/v1/chat/completions", {"messages": []})[::3] == \
               (400, _error("messages must contain at least one item"))
        # generation needs the GPU; without one the session's error is the answer: status 400, or, once the
        # event stream has begun, an error event and [DONE] (serve.rs:976-985)
        status, _, _, body = srv.request("POST", "/v1/completions", {"prompt_ids": [1, 2, 3], "max_tokens": 2})
        if status != 200:
            assert status == 400 and body["error"]["message"].startswith("failed to initialize hip decode")
            headers, events, done = srv.events("/v1/chat/completions", {"messages": [{"role": "user", "content_ids": [1, 2]}],
                                                                        "stream": True})
            assert headers["Content-Type"] == "text/event-stream" and done
            assert events[0]["choices"][0]["delta"] == {"role": "assistant"}
            assert events[1:] == [body]
        # a request line alone is answered too (no headers, no body)
        s = socket.create_connection(("127.0.0.1", srv.port), timeout=10)
        s.sendall(b"GET /healthz\n\n")
        assert s.makefile("rb").read().startswith(b"HTTP/1.1 200 OK\r\n")
        s.close()
        s = socket.create_connection(("127.0.0.1", srv.port), timeout=10)
        s.sendall(b"\r\n\r\n")
        assert b'"message":"empty request"' in s.makefile("rb").read()
        s.close()
        assert srv.proc.poll() is None
    finally:
        srv.close()


def test_command_line():
    def run(*args):
        return subprocess.run([SERVE] + list(args), capture_output=True, text=True, timeout=30)

    p = run()
    assert p.returncode == 1 and p.stderr.startswith("--checkpoint required") and "Usage: serve" in p.stderr
    p = run("--frobnicate")
    assert p.returncode == 1 and p.stderr.startswith("Unknown arg: --frobnicate")
    p = run("--model", "bench_tiny", "--decode-backend", "cuda")
    assert p.returncode == 2 and "--decode-backend must be one of: auto, naive, hip" in p.stderr
    p = run("--model", "bench_tiny", "--tokenizer", "tok.json")
    assert p.returncode == 2 and "tokenizer" in p.stderr
    p = run("--checkpoint", "/nonexistent/ckpt.bin")
    assert p.returncode == 2 and "failed to load checkpoint" in p.stderr
    p = run("--model", "bench_tiny", "--bind", "nowhere")
    assert p.returncode == 2 and "--bind must be HOST:PORT" in p.stderr
    assert run("--help").returncode == 0


# ---------------------------------------------------------------- on the GPU: answers equal direct session-cache calls
META_KEYS = ["effective_prompt_tokens", "prompt_truncated", "cache_prefix_tokens", "cache_hit", "base_prefill_ms",
             "request_prefill_ms", "total_prefill_ms", "decode_ms_total", "decode_ms_avg", "total_ms"]


@pytest.mark.gpu
def test_completions_equal_direct_cache_calls(tmp_path):
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w = synth.make_weights(cfg, seed=8, std=0.08, round_bf16=True)
    path = tmp_path / "ckpt_000003.bin"
    engine.write_checkpoint(path, cfg, w, step=3)
    srv = Server(["--checkpoint", str(path), "--decode-backend", "hip", "--weight-dtype", "bf16", "--max-cache-sessions", "3"])
    cache = engine.SessionCache(cfg, w, max_entries=3, weight_dtype=1, kv_dtype=0)
    try:
        base = [1, 2, 3, 4, 5, 6, 7, 8, 9]
        longer = base + [11, 12, 13]
        window = list(range(1, 121))                         # longer than seq: the last 96 ids count
        requests = [({"prompt_ids": base, "max_tokens": 6}, engine.GenerationRequest(HIP, steps=6)),
                    ({"prompt_ids": base, "max_tokens": 6}, engine.GenerationRequest(HIP, steps=6)),
                    ({"prompt_ids": longer, "max_tokens": 5, "temperature": 0.8, "top_k": 4, "n": 2, "seed": 5},
                     engine.GenerationRequest(HIP, steps=5, temperature=0.8, top_k=4, samples=2, seed=5)),
                    ({"prompt_ids": base, "max_tokens": 4, "decode_backend": "naive"}, engine.GenerationRequest(NAIVE, steps=4)),
                    ({"prompt_ids": window, "max_tokens": 3}, engine.GenerationRequest(HIP, steps=3))]
        for i, (body, req) in enumerate(requests):
            status, _, _, got = srv.request("POST", "/v1/completions", body)
            assert status == 200, got
            want = cache.generate(body["prompt_ids"], req)
            assert list(got) == ["id", "object", "created", "model", "choices", "usage", "rustane"]
            assert got["object"] == "text_completion" and got["model"] == "rustane" and got["id"].startswith("cmpl-")
            assert abs(got["created"] - time.time()) < 600
            assert len(got["choices"]) == len(want.batch.results)
            for k, (c, r) in enumerate(zip(got["choices"], want.batch.results)):
                assert list(c) == ["index", "text", "finish_reason", "generated_ids", "full_sequence"]
                assert (c["index"], c["text"], c["finish_reason"]) == (k, "", "length")
                assert c["generated_ids"] == list(map(int, r.sampled)) and c["full_sequence"] == list(map(int, r.generated))
            n_prompt, n_new = len(body["prompt_ids"]), body["max_tokens"]
            assert got["usage"] == {"prompt_tokens": n_prompt, "completion_tokens": n_new, "total_tokens": n_prompt + n_new}
            meta = got["rustane"]
            assert list(meta) == META_KEYS
            assert (meta["effective_prompt_tokens"], meta["prompt_truncated"], meta["cache_prefix_tokens"], meta["cache_hit"]) == \
                   (want.effective_prompt_tokens, want.prompt_truncated, want.cache_prefix_tokens, want.cache_prefix_tokens > 0)
            assert all(isinstance(meta[k], float) and meta[k] >= 0 for k in META_KEYS[4:])
        # what the five requests did to the cache: new session, exact hit, prefix hit + own entry, exact hit, new (truncated)
        metas = [srv.request("POST", "/v1/completions", b)[3]["rustane"] for b, _ in requests[:1]]
        assert metas[0]["cache_hit"] and metas[0]["cache_prefix_tokens"] == len(base) and metas[0]["request_prefill_ms"] == 0
        health = srv.request("GET", "/healthz")[3]
        assert health["cache_entries"] == len(cache) == 3 and health["max_cache_sessions"] == 3
        # no tokens asked for: the prompt is prefilled (here: found in the cache) and nothing is generated
        status, _, _, got = srv.request("POST", "/v1/completions", {"prompt_ids": base, "max_tokens": 0})
        assert status == 200 and got["choices"][0]["generated_ids"] == [] and got["choices"][0]["full_sequence"] == base
        assert got["usage"] == {"prompt_tokens": 9, "completion_tokens": 0, "total_tokens": 9}
    finally:
        srv.close()
        cache.close()


@pytest.mark.gpu
def test_streams_and_chat(tmp_path):
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w = synth.make_weights(cfg, seed=9, std=0.08, round_bf16=True)
    path = tmp_path / "ckpt_000001.bin"
    engine.write_checkpoint(path, cfg, w, step=1)
    srv = Server(["--checkpoint", str(path), "--decode-backend", "hip", "--weight-dtype", "bf16", "--kv-dtype", "bf16",
                  "--model-name", "chatty"])
    cache = engine.SessionCache(cfg, w, max_entries=32, weight_dtype=1, kv_dtype=1)
    try:
        prompt = [3, 1, 4, 1, 5, 9, 2, 6]
        req = engine.GenerationRequest(HIP, steps=7, temperature=0.9, top_k=5, seed=11)
        want = cache.generate(prompt, req).batch.results[0]
        body = {"prompt_ids": prompt, "max_tokens": 7, "temperature": 0.9, "top_k": 5, "seed": 11, "stream": True}
        headers, events, done = srv.events("/v1/completions", body)
        assert headers["Content-Type"] == "text/event-stream" and headers["Transfer-Encoding"] == "chunked"
        assert headers["Cache-Control"] == "no-cache" and done
        assert len(events) == 8                               # one event per token and the closing one
        ids = []
        for e in events[:-1]:
            assert list(e) == ["id", "object", "created", "model", "choices"] and e["object"] == "text_completion"
            (c,) = e["choices"]
            assert list(c) == ["index", "text", "finish_reason", "generated_ids"]
            assert (c["index"], c["text"], c["finish_reason"]) == (0, "", None) and len(c["generated_ids"]) == 1
            ids += c["generated_ids"]
        assert ids == list(map(int, want.sampled))
        last = events[-1]
        assert list(last) == ["id", "object", "created", "model", "choices", "rustane"] and list(last["rustane"]) == META_KEYS
        assert last["choices"] == [{"index": 0, "text": "", "finish_reason": "length", "generated_ids": []}]
        assert len({e["id"] for e in events}) == 1 and events[0]["id"].startswith("cmpl-") and events[0]["model"] == "chatty"
        assert last["rustane"]["cache_hit"] is False and last["rustane"]["effective_prompt_tokens"] == len(prompt)

        # the same prompt as a chat: ids of the messages joined; answered from the cached session
        chat = {"model": "chatty", "messages": [{"role": "system", "content_ids": prompt[:3]}, {"role": "user", "content_ids": prompt[3:]}],
                "max_tokens": 7, "temperature": 0.9, "top_k": 5, "seed": 11}
        status, _, _, got = srv.request("POST", "/v1/chat/completions", chat)
        assert status == 200 and list(got) == ["id", "object", "created", "model", "choices", "usage", "rustane"]
        assert got["object"] == "chat.completion" and got["id"].startswith("chatcmpl-")
        (c,) = got["choices"]
        assert list(c) == ["index", "message", "finish_reason", "generated_ids", "full_sequence"]
        assert c["message"] == {"role": "assistant", "content": ""} and c["finish_reason"] == "length"
        assert c["generated_ids"] == list(map(int, want.sampled)) and c["full_sequence"] == list(map(int, want.generated))
        assert got["rustane"]["cache_hit"] and got["rustane"]["cache_prefix_tokens"] == len(prompt)
        assert got["usage"] == {"prompt_tokens": 8, "completion_tokens": 7, "total_tokens": 15}

        headers, events, done = srv.events("/v1/chat/completions", dict(chat, stream=True))
        assert done and len(events) == 9                      # role, one per token, closing
        assert all(e["object"] == "chat.completion.chunk" and e["id"].startswith("chatcmpl-") for e in events)
        assert events[0]["choices"] == [{"index": 0, "delta": {"role": "assistant"}, "finish_reason": None, "generated_ids": []}]
        assert [e["choices"][0]["delta"] for e in events[1:-1]] == [{"content": ""}] * 7
        assert sum((e["choices"][0]["generated_ids"] for e in events[1:-1]), []) == list(map(int, want.sampled))
        assert events[-1]["choices"] == [{"index": 0, "delta": {}, "finish_reason": "length", "generated_ids": []}]
        assert events[-1]["rustane"]["cache_hit"] and "rustane" not in events[1]

        # a stream of no tokens is its closing event
        headers, events, done = srv.events("/v1/completions", {"prompt_ids": prompt, "max_tokens": 0, "stream": True})
        assert done and len(events) == 1 and events[0]["choices"][0]["finish_reason"] == "length"
        assert srv.request("GET", "/healthz")[3]["cache_entries"] == 1
    finally:
        srv.close()
        cache.close()


@pytest.mark.gpu
def test_server_over_a_converted_checkpoint(tmp_path):
    # the server loads a checkpoint converted ahead of time (4-bit weights as the device stores them) with no flag
    # naming the format; its answers are those of a cache built from the fp32 arrays in that format
    cfg = Config.make(dim=256, hidden=640, heads=2, hd=128, seq=96, nlayers=2, vocab=320)
    w = synth.make_weights(cfg, seed=14, std=0.08, round_bf16=False)
    src, dst = tmp_path / "ckpt_000002.bin", tmp_path / "ckpt_000002.rstq"
    engine.write_checkpoint(src, cfg, w, step=2)
    gen = os.path.join(ROOT, "rustane_amd", "lib", "generate")
    p = subprocess.run([gen, "--checkpoint", str(src), "--weight-dtype", "int4", "--convert-to", str(dst)],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    srv = Server(["--checkpoint", str(dst), "--decode-backend", "hip"])
    cache = engine.SessionCache(cfg, w, max_entries=4, weight_dtype=3, kv_dtype=0)
    try:
        prompt = [7, 8, 9, 10, 11, 12]
        for body, req in (({"prompt_ids": prompt, "max_tokens": 9}, engine.GenerationRequest(HIP, steps=9)),
                          ({"prompt_ids": prompt + [1, 2], "max_tokens": 6, "temperature": 0.7, "top_k": 5, "seed": 3},
                           engine.GenerationRequest(HIP, steps=6, temperature=0.7, top_k=5, seed=3))):
            status, _, _, got = srv.request("POST", "/v1/completions", body)
            assert status == 200, got
            want = cache.generate(body["prompt_ids"], req).batch.results[0]
            assert got["choices"][0]["generated_ids"] == list(map(int, want.sampled))
    finally:
        srv.close()
        cache.close()
