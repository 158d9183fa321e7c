"""Host tests of the OpenAI-compatible engine shim (eidola_amd/engine_shim.py), in the style of
the reference's fake-engine tests (/root/reference/crates/eidola-app-core/tests/local_models.rs:
855-861): the shim is started the way the reference starts its engine (same flags, polled on
/health) with the CPU echo engine behind it, and answers the body the reference sends."""
import json
import os
import socket
import subprocess
import sys
import threading
import time
import urllib.error
import urllib.request

import pytest

from eidola_amd import engine_shim as shim

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def reference_body(model, messages, max_completion_tokens, stream=False, include_usage=False):
    """The outer shape of chat_completion_request_body (eidola-common/src/lib.rs:116-139)."""
    body = {"model": model, "messages": messages, "max_completion_tokens": max_completion_tokens}
    if stream:
        body["stream"] = True
        if include_usage:
            body["stream_options"] = {"include_usage": True}
    return body


def post(port, body, raw=False):
    data = body if isinstance(body, bytes) else json.dumps(body).encode()
    req = urllib.request.Request(f"http://127.0.0.1:{port}/v1/chat/completions", data=data,
                                 headers={"Content-Type": "application/json"})
    with urllib.request.urlopen(req, timeout=10) as r:
        payload = r.read()
        return (r.status, r.headers, payload) if raw else json.loads(payload)


@pytest.fixture()
def server():
    srv = shim.make_server("127.0.0.1", 0, shim.FakeEngine(), "local/test-model")
    t = threading.Thread(target=srv.serve_forever, daemon=True)
    t.start()
    yield srv.server_address[1]
    srv.shutdown()
    srv.server_close()


def test_flags_of_the_reference_are_accepted():
    a = shim.parse_args(["-m", "/models/x.gguf", "--host", "127.0.0.1", "--port", "18080", "--alias",
                         "local/x", "-c", "8192", "-ngl", "999", "--jinja", "--no-webui"])
    assert (a.model, a.host, a.port, a.alias, a.ctx_size, a.n_gpu_layers) == \
        ("/models/x.gguf", "127.0.0.1", 18080, "local/x", 8192, 999)
    assert a.jinja and a.no_webui and a.engine == "synthetic"


def test_health_and_models(server):
    with urllib.request.urlopen(f"http://127.0.0.1:{server}/health", timeout=5) as r:
        assert r.status == 200 and json.loads(r.read()) == {"status": "ok"}
    with urllib.request.urlopen(f"http://127.0.0.1:{server}/v1/models", timeout=5) as r:
        assert json.loads(r.read())["data"][0]["id"] == "local/test-model"
    with pytest.raises(urllib.error.HTTPError) as e:
        urllib.request.urlopen(f"http://127.0.0.1:{server}/nope", timeout=5)
    assert e.value.code == 404


def test_blocking_completion_has_the_openai_shape(server):
    msgs = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "abc déf"}]
    r = post(server, reference_body("local/test-model", msgs, 64))
    assert r["object"] == "chat.completion" and r["model"] == "local/test-model"
    c = r["choices"][0]
    assert c["index"] == 0 and c["finish_reason"] == "stop"
    assert c["message"] == {"role": "assistant", "content": "féd cba"}
    u = r["usage"]
    assert u["prompt_tokens"] == len(shim.render_prompt(msgs))
    assert u["total_tokens"] == u["prompt_tokens"] + u["completion_tokens"]
    # the budget cuts the answer: finish_reason says so
    r = post(server, reference_body("m", [{"role": "user", "content": "0123456789"}], 4))
    assert r["choices"][0] == {"index": 0, "finish_reason": "length",
                               "message": {"role": "assistant", "content": "9876"}}


def test_streaming_completion_is_sse_with_usage_and_done(server):
    status, headers, payload = post(server, reference_body("m", [{"role": "user", "content": "héllo"}], 32,
                                                           stream=True, include_usage=True), raw=True)
    assert status == 200 and headers["Content-Type"].startswith("text/event-stream")
    events = [e[len(b"data: "):] for e in payload.split(b"\n\n") if e.startswith(b"data: ")]
    assert events[-1] == b"[DONE]"
    chunks = [json.loads(e) for e in events[:-1]]
    assert all(c["object"] == "chat.completion.chunk" for c in chunks)
    assert chunks[0]["choices"][0]["delta"]["role"] == "assistant"
    text = "".join(c["choices"][0]["delta"].get("content", "") for c in chunks if c["choices"])
    assert text == "olléh"
    assert chunks[-2]["choices"][0]["finish_reason"] == "stop" and chunks[-2]["choices"][0]["delta"] == {}
    assert chunks[-1]["choices"] == [] and chunks[-1]["usage"]["completion_tokens"] == len("olléh".encode())
    # without stream_options there is no usage chunk
    _, _, payload = post(server, reference_body("m", [{"role": "user", "content": "x"}], 8, stream=True), raw=True)
    assert b'"usage"' not in payload and payload.rstrip().endswith(b"data: [DONE]")


@pytest.mark.parametrize("body", [b"{not json", json.dumps({"model": "m"}).encode(),
                                  json.dumps({"messages": [], "max_completion_tokens": 4}).encode(),
                                  json.dumps({"messages": [{"role": "user", "content": "x"}],
                                              "max_completion_tokens": 0}).encode()])
def test_bad_requests_get_a_400_with_an_error_object(server, body):
    with pytest.raises(urllib.error.HTTPError) as e:
        post(server, body)
    assert e.value.code == 400
    assert json.loads(e.value.read())["error"]["type"] == "invalid_request_error"


class _FailingEngine:
    """Yields two tokens, then fails the way a GPU step would."""
    name = "failing"

    def generate(self, prompt_ids, max_new_tokens):
        yield ord("o")
        yield ord("k")
        raise RuntimeError("step failed")


def test_an_engine_failure_is_a_500_or_an_error_event_and_the_server_lives_on():
    srv = shim.make_server("127.0.0.1", 0, _FailingEngine(), "local/test-model")
    threading.Thread(target=srv.serve_forever, daemon=True).start()
    port = srv.server_address[1]
    try:
        msgs = [{"role": "user", "content": "x"}]
        with pytest.raises(urllib.error.HTTPError) as e:
            post(port, reference_body("m", msgs, 8))
        assert e.value.code == 500 and json.loads(e.value.read())["error"]["type"] == "server_error"
        status, _, payload = post(port, reference_body("m", msgs, 8, stream=True), raw=True)
        assert status == 200 and b'"content": "o"' in payload and b'"content": "k"' in payload
        assert b'"server_error"' in payload
        assert payload.rstrip().endswith(b"data: [DONE]")
        with urllib.request.urlopen(f"http://127.0.0.1:{port}/health", timeout=5) as r:
            assert r.status == 200
    finally:
        srv.shutdown()
        srv.server_close()


def test_started_and_polled_the_way_the_reference_does():
    """The reference spawns the engine with its flags, stdin/stdout null, and polls /health
    until it answers 2xx (local_models.rs:1612-1626, 2020-2063)."""
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    child = subprocess.Popen(
        [sys.executable, "-m", "eidola_amd.engine_shim", "-m", "/nonexistent/model.gguf", "--host",
         "127.0.0.1", "--port", str(port), "--alias", "local/echo", "-c", "4096", "-ngl", "999", "--jinja",
         "--no-webui", "--engine", "fake"],
        cwd=ROOT, stdin=subprocess.DEVNULL, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
    try:
        deadline, ready = time.time() + 30, False
        while time.time() < deadline and child.poll() is None:
            try:
                with urllib.request.urlopen(f"http://127.0.0.1:{port}/health", timeout=1) as r:
                    ready = 200 <= r.status < 300
                    break
            except (urllib.error.URLError, ConnectionError, socket.timeout):
                time.sleep(0.1)
        assert ready, child.stderr.read().decode() if child.poll() is not None else "never became ready"
        r = post(port, reference_body("local/echo", [{"role": "user", "content": "ping"}], 16))
        assert r["choices"][0]["message"]["content"] == "gnip" and r["model"] == "local/echo"
    finally:
        child.terminate()
        child.wait(timeout=10)


# ---- the batching loop on the host: the real scheduler, a stubbed forward (no GPU) ----------
def stub_engine(ctx=64, num_blocks=None, max_seqs=4, answer=ord("a")):
    """SyntheticAttentionEngine without its device side: forward() votes for one byte."""
    import torch
    eng = shim.SyntheticAttentionEngine(layers=1, ctx=ctx, num_blocks=num_blocks, max_seqs=max_seqs,
                                        chunk=16, step_tokens=32, device=None)
    eng.forward_calls = []

    def forward(seq_ids, token_lists):
        q_lens = [len(t) for t in token_lists]
        eng.sched.build_batch(seq_ids, q_lens)     # raises on a request the pool cannot hold
        eng.forward_calls.append((list(seq_ids), q_lens))
        logits = torch.zeros((len(seq_ids), shim.VOCAB))
        logits[:, answer] = 1.0
        return logits
    eng.forward = forward
    return eng


@pytest.mark.parametrize("max_new", [64, 65, 4096])   # == ctx, > ctx, the reference's usual 4096
def test_a_budget_of_the_whole_context_keeps_the_tail_of_a_long_prompt(max_new):
    """The reference sends max_completion_tokens = min(context_length, 4096)
    (/root/reference/crates/eidola-app-core/src/lib.rs:5595), which is the engine's -c: the
    budget shrinks to the context, the prompt to its tail, and nothing outgrows its table row."""
    eng = stub_engine(ctx=64)
    prompt = list(range(1, 200))                      # longer than the context
    out = list(eng.generate(prompt, max_new))
    assert out == [ord("a")] * 63                     # ctx - 1 new tokens behind one prompt token
    fed = sum(q for _, qs in eng.forward_calls for q in qs)
    assert fed == 1 + 62                              # one prompt token, then 62 decode rows (the last token is not fed back)
    assert eng.sched.free_blocks == eng.num_blocks and eng.committed == 0


def test_a_long_prompt_with_a_small_budget_keeps_its_latest_tokens():
    eng = stub_engine(ctx=64)
    seen = []
    real = eng.forward

    def forward(seq_ids, token_lists):
        seen.extend(t for ts in token_lists for t in ts if len(ts) > 1 or not seen)
        return real(seq_ids, token_lists)
    eng.forward = forward
    prompt = list(range(1, 200))
    assert list(eng.generate(prompt, 4)) == [ord("a")] * 4
    assert seen[:60] == prompt[-60:]                  # ctx - 4 prompt tokens: the tail


def test_a_request_the_pool_can_never_hold_is_refused_and_the_engine_goes_on():
    """A request needing more pages than the pool has used to sit at the head of the queue
    for ever, with the stepping thread spinning on an empty batch behind it."""
    eng = stub_engine(ctx=256, num_blocks=4, max_seqs=2)   # 4 pages = 64 tokens in all
    with pytest.raises(RuntimeError, match="KV pages"):
        list(eng.generate(list(range(1, 100)), 100))
    assert not eng.waiting and not eng.active
    assert list(eng.generate([1, 2, 3], 5)) == [ord("a")] * 5   # the next request is served
    assert eng.sched.free_blocks == 4


def test_concurrent_requests_wait_for_pages_and_all_finish():
    eng = stub_engine(ctx=64, num_blocks=6, max_seqs=4)   # two requests of 3 pages fit at a time
    results = {}

    def run(i):
        results[i] = list(eng.generate(list(range(1, 30)), 10))
    threads = [threading.Thread(target=run, args=(i,)) for i in range(5)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=30)
    assert all(results.get(i) == [ord("a")] * 10 for i in range(5))
    assert eng.max_step_seqs <= 2 and eng.sched.free_blocks == 6 and eng.committed == 0


def test_tools_in_the_request_are_accepted_and_ignored(server):
    """`tools` is part of the reference's request body
    (/root/reference/crates/eidola-common/src/lib.rs:129-131); this engine answers in plain text."""
    body = reference_body("m", [{"role": "user", "content": "abc"}], 16)
    body["tools"] = [{"type": "function", "function": {"name": "f", "parameters": {"type": "object"}}}]
    resp = post(server, body)
    assert resp["choices"][0]["message"]["content"] == "cba"
    body["tools"] = "not a list"
    with pytest.raises(urllib.error.HTTPError) as ei:
        post(server, body)
    assert ei.value.code == 400 and "tools" in json.loads(ei.value.read())["error"]["message"]
