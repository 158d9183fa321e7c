"""The synthetic attention engine behind the OpenAI shim on the GPU: the scheduler, the fused
QKV + RoPE + KV write, chunked prefill, decode and the output projection chained per generated
token.  Checks: decoding token by token lands on the same logits as one prefill pass over the
same tokens (the KV cache the decode steps built equals what a prefill writes, and the decode
and prefill kernels agree), sequences that share a step (prefill chunks beside decode rows in
one ragged call) do not see each other, generation is deterministic, concurrent requests are
batched into shared steps, and an HTTP round trip works."""
import json
import threading
import urllib.request

import numpy as np
import pytest
import torch

from eidola_amd import engine_shim as shim

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def engine():
    return shim.SyntheticAttentionEngine(layers=3, ctx=1024, seed=7)


def test_decode_steps_agree_with_one_prefill_pass(engine):
    prompt = shim.render_prompt([{"role": "user", "content": "the quick brown fox jumps over the lazy dog " * 5}])
    assert len(prompt) > 200                      # more than one 64-key chunk, beyond the 128-token window
    extra = [104, 105, 33, 10, 200, 7, 99, 32]    # tokens appended one decode step at a time
    engine.sched.add_seq(1001)
    logits = engine.forward([1001], [prompt])[0]  # chunked-prefill path (eid_attn_varlen, > 64 rows)
    for t in extra:
        logits = engine.forward([1001], [[t]])[0]  # decode path (fused QKV + write, eid_attn_decode)
    engine.sched.add_seq(1002)
    ref = engine.forward([1002], [prompt + extra])[0]  # everything as one prefill chunk
    engine.sched.free_seq(1001)
    engine.sched.free_seq(1002)
    a, b = logits.double().cpu().numpy(), ref.double().cpu().numpy()
    assert np.isfinite(a).all() and np.isfinite(b).all()
    cos = float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))
    assert cos > 0.9995, cos
    assert np.abs(a - b).max() < 0.05 * np.abs(b).std() + 0.5, (np.abs(a - b).max(), b.std())
    assert int(a[:257].argmax()) == int(b[:257].argmax())


def _close(a, b):
    a, b = a.double().cpu().numpy(), b.double().cpu().numpy()
    assert np.isfinite(a).all() and np.isfinite(b).all()
    cos = float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))
    assert cos > 0.9995, cos
    assert np.abs(a - b).max() < 0.05 * np.abs(b).std() + 0.5, (np.abs(a - b).max(), b.std())


def test_sequences_that_share_a_step_do_not_see_each_other(engine):
    """A decode row, a prefill chunk and a longer prefill chunk in ONE step (one ragged
    eid_attn_varlen call per layer) against each sequence stepped alone."""
    rng = np.random.default_rng(3)
    prompts = [list(rng.integers(0, 256, size=n)) for n in (150, 40, 300)]
    nxt = [int(rng.integers(0, 256)), list(rng.integers(0, 256, size=70)), list(rng.integers(0, 256, size=200))]
    alone = []
    for i, (p0, more) in enumerate(zip(prompts, nxt)):           # each sequence by itself
        sid = 2001 + i
        engine.sched.add_seq(sid)
        engine.forward([sid], [p0])
        alone.append(engine.forward([sid], [[more] if isinstance(more, int) else more])[0])
        engine.sched.free_seq(sid)
    ids = [2011, 2012, 2013]
    for sid in ids:
        engine.sched.add_seq(sid)
    engine.forward(ids, prompts)                                   # three prefill chunks in one step
    mixed = engine.forward(ids, [[nxt[0]], nxt[1], nxt[2]])       # decode row + two prefill chunks
    for sid in ids:
        engine.sched.free_seq(sid)
    for i in range(3):
        _close(mixed[i], alone[i])


def test_concurrent_requests_are_batched_into_shared_steps(engine):
    prompts = [shim.render_prompt([{"role": "user", "content": "request %d " % i + "lorem ipsum " * (3 + 9 * i)}])
               for i in range(6)]
    free0, steps0 = engine.sched.free_blocks, engine.steps
    engine.max_step_seqs = 0
    outs = [None] * len(prompts)

    def run(i):
        outs[i] = list(engine.generate(prompts[i], 10))
    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(prompts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert all(o is not None and 1 <= len(o) <= 10 and all(0 <= t <= shim.EOS for t in o) for o in outs)
    assert engine.max_step_seqs >= 2                 # requests did share steps
    assert engine.steps - steps0 < sum(len(o) + 1 for o in outs)   # fewer steps than one at a time
    assert engine.sched.free_blocks == free0 and not engine.active and not engine.waiting


def test_requests_wait_for_pages_instead_of_failing():
    """A pool too small for all requests at once: admission waits until the running ones have
    returned their pages; every request completes."""
    eng = shim.SyntheticAttentionEngine(layers=2, ctx=512, seed=5, num_blocks=40, max_seqs=8)
    prompts = [list(range(1, 200)) for _ in range(5)]           # 199 + 8 tokens -> 13 pages each
    outs = [None] * len(prompts)

    def run(i):
        outs[i] = list(eng.generate(prompts[i], 8))
    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(prompts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert all(o is not None and 1 <= len(o) <= 8 for o in outs)
    assert eng.max_step_seqs <= 3 and eng.committed == 0 and eng.sched.free_blocks == 40


def test_generation_is_deterministic_and_frees_its_blocks(engine):
    prompt = shim.render_prompt([{"role": "user", "content": "hello"}])
    free0 = engine.sched.free_blocks
    first = list(engine.generate(prompt, 12))
    again = list(engine.generate(prompt, 12))
    assert first == again and 1 <= len(first) <= 12
    assert all(0 <= t <= shim.EOS for t in first)
    assert engine.sched.free_blocks == free0


def test_http_round_trip_on_the_gpu_engine(engine):
    srv = shim.make_server("127.0.0.1", 0, engine, "local/synthetic")
    threading.Thread(target=srv.serve_forever, daemon=True).start()
    try:
        port = srv.server_address[1]
        body = {"model": "local/synthetic", "messages": [{"role": "user", "content": "ping"}],
                "max_completion_tokens": 6}
        req = urllib.request.Request(f"http://127.0.0.1:{port}/v1/chat/completions",
                                     data=json.dumps(body).encode(), headers={"Content-Type": "application/json"})
        with urllib.request.urlopen(req, timeout=60) as r:
            out = json.loads(r.read())
        assert out["object"] == "chat.completion" and out["choices"][0]["finish_reason"] in ("stop", "length")
        assert out["usage"]["completion_tokens"] <= 6
        torch.cuda.synchronize()
    finally:
        srv.shutdown()
        srv.server_close()
