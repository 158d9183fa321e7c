"""OpenAI-compatible engine shim over the paged sink-attention path.

The reference's only seam toward an inference engine is a child process that speaks
OpenAI-compatible HTTP: it starts `llama-server -m <file> --host 127.0.0.1 --port <p>
--alias <id> -c <ctx> -ngl 999 --jinja --no-webui`
(/root/reference/crates/eidola-app-core/src/local_models.rs:1612-1626), polls `GET /health`
until it answers 2xx (local_models.rs:2020-2063) and then posts the body built by
`chat_completion_request_body` (/root/reference/crates/eidola-common/src/lib.rs:116-139:
`model`, `messages`, `max_completion_tokens`, optional `tools`, `stream`,
`stream_options.include_usage`) to `/v1/chat/completions`.

This module is the smallest process that honours that contract on top of this package:
the same flags, `/health`, `/v1/models`, blocking and SSE chat completions.  What it runs
behind them is a SYNTHETIC model: gpt-oss-shaped attention blocks (QKV projection, rotary
embedding, paged KV cache managed by eidola_amd.Scheduler, sink attention through the HIP
kernels, output projection, residual) with seeded random weights, a byte-level tokenizer and
greedy sampling.  No checkpoint is read (none exists on the box), there is no MLP / MoE and
no learned norm, so the text it produces is deterministic noise; the request handling, the
continuous batching of concurrent requests through the scheduler (prefill chunks and decode
rows of different requests in one ragged attention call per layer) and the kernels per
generated token are real.
`--engine fake` swaps the model for a CPU echo so the HTTP layer can be tested anywhere.
"""
import argparse
import json
import queue
import threading
import time
import uuid
from http.server import BaseHTTPRequestHandler, ThreadingHTTPServer

EOS = 256           # byte-level vocabulary: 0..255 are bytes, 256 ends a turn
VOCAB = 320         # padded to a multiple of 64 for the projection kernels


def render_prompt(messages):
    """Chat template of the synthetic model: `<|role|>content<|end|>` per message, then the
    assistant header; everything as UTF-8 bytes."""
    parts = []
    for msg in messages:
        content = msg.get("content")
        if isinstance(content, list):   # OpenAI content parts: keep the text ones
            content = "".join(p.get("text", "") for p in content if isinstance(p, dict))
        parts.append(f"<|{msg.get('role', 'user')}|>{content or ''}<|end|>")
    parts.append("<|assistant|>")
    return list("".join(parts).encode("utf-8"))


class FakeEngine:
    """CPU stand-in: answers with the last user message reversed, one byte per token."""
    name = "fake"

    def generate(self, prompt_ids, max_new_tokens):
        """Yields byte tokens; EOS when the answer is complete, nothing more when the budget
        of `max_new_tokens` ran out first."""
        text = bytes(prompt_ids).decode("utf-8", "replace")
        last = text.rsplit("<|user|>", 1)[-1].split("<|end|>", 1)[0]
        answer = last[::-1].encode("utf-8")
        for b in answer[:max_new_tokens]:
            yield b
        if len(answer) <= max_new_tokens:
            yield EOS


class _Request:
    """One generation in flight inside SyntheticAttentionEngine."""

    def __init__(self, seq_id, prompt_ids, max_new_tokens):
        self.seq_id, self.prompt, self.budget = seq_id, prompt_ids, max_new_tokens
        self.blocks = (len(prompt_ids) + max_new_tokens + 15) // 16   # pages it may come to hold
        # (generate() has cut prompt and budget to the context: at most max_blocks_per_seq)
        self.fed = 0              # prompt tokens already in the KV cache
        self.last = None          # the sampled token to feed next
        self.produced = 0
        self.out = queue.Queue()  # tokens, then _DONE (or an exception to re-raise)


_DONE = object()


class SyntheticAttentionEngine:
    """Attention-only stack with seeded random weights on cuda:0 behind a continuous-batching
    loop: requests from any number of HTTP threads join a shared step (up to `max_seqs`
    sequences), in which sequences still reading their prompt contribute a prefill chunk and
    the others one decode row; the scheduler builds the ragged batch and every layer's
    attention is ONE eid_attn_varlen call over it (eid_attn_decode when every row is a decode
    row)."""
    name = "synthetic"

    def __init__(self, layers=4, ctx=4096, seed=0, num_blocks=None, max_seqs=16, chunk=512,
                 step_tokens=2048, device="cuda:0"):
        """`device=None` builds the host side only (scheduler, queues, the batching loop) and
        leaves `forward` to the caller: the loop can then be tested without a GPU."""
        import numpy as np
        import torch
        import eidola_amd as ea
        self.np, self.torch, self.ea = np, torch, ea
        ea.load_library()
        dev = device
        self.dev, self.layers, self.ctx = dev, layers, ctx
        self.max_seqs, self.chunk, self.step_tokens = max_seqs, chunk, step_tokens
        self.H, self.NQKV = 2880, (64 + 2 * 8) * 64
        self.geoms = [ea.AttnGeometry(window=128 if l % 2 == 0 else 0) for l in range(layers)]
        self.max_blocks = (ctx + 15) // 16
        self.num_blocks = num_blocks or (max_seqs + 1) * self.max_blocks
        self.sched = ea.Scheduler(self.num_blocks, self.max_blocks)
        self.cv = threading.Condition()
        self.waiting, self.active = [], []
        self.committed = 0        # pages the active requests may come to hold between them
        self.next_id = 1
        self.steps = self.mixed_steps = self.max_step_seqs = 0   # (for tests and curiosity)
        self.worker = None
        if dev is None:
            return
        g = torch.Generator(device=dev).manual_seed(seed)
        rnd = lambda *shape, scale: (torch.randn(shape, device=dev, generator=g) * scale).to(torch.bfloat16)
        self.emb = rnd(VOCAB, self.H, scale=1.0)
        self.wqkv = [rnd(self.NQKV, self.H, scale=0.02) for _ in range(layers)]
        self.wo = [rnd(self.H, 4096, scale=0.02) for _ in range(layers)]
        self.sinks = [torch.randn(64, device=dev, generator=g) for _ in range(layers)]
        self.kc = [torch.zeros((self.num_blocks, 16, 8, 64), dtype=torch.bfloat16, device=dev)
                   for _ in range(layers)]
        self.vc = [torch.zeros_like(k) for k in self.kc]
        self.cos_sin = torch.from_numpy(ea.yarn_cos_sin(ctx + 1)).to(dev)

    def _norm(self, h):
        x = h.float()
        return (x * self.torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).to(self.torch.bfloat16)

    def forward(self, seq_ids, token_lists):
        """Appends token_lists[i] to sequence seq_ids[i] (a prefill chunk or one decode token
        each) and returns the logits of every sequence's last position, fp32 [len(seq_ids), VOCAB]."""
        torch, ea = self.torch, self.ea
        q_lens = [len(t) for t in token_lists]
        T = sum(q_lens)
        b = self.sched.build_batch(seq_ids, q_lens)
        to_dev = lambda a: torch.from_numpy(a).to(self.dev)
        bt, slots, cu, sl, pos = (to_dev(b.block_table), to_dev(b.slot_mapping), to_dev(b.cu_seqlens_q),
                                  to_dev(b.seq_lens), to_dev(b.positions))
        hidden = self.emb[torch.tensor([t for ts in token_lists for t in ts], device=self.dev)].clone()
        for l in range(self.layers):
            g, x = self.geoms[l], self._norm(hidden)
            if T <= 64:   # projection, rotary embedding, split and KV write in one launch
                q = ea.qkv_rope_kv_write(g, x, self.wqkv[l], None, pos, self.cos_sin, self.kc[l], self.vc[l], slots)
            else:
                qkv = ea.o_proj(x, self.wqkv[l])
                q = ea.rope_kv_write(g, qkv, pos, self.cos_sin, self.kc[l], self.vc[l], slots)
            if b.max_q_len == 1:
                out = ea.attn_decode(g, q, self.kc[l], self.vc[l], bt, sl, max_kv_len=b.max_kv_len,
                                     sinks=self.sinks[l], sum_kv_len=b.sum_kv_len, seq_lens_host=b.seq_lens,
                                     block_table_host=b.block_table)
            else:
                out = ea.attn_varlen(g, q, self.kc[l], self.vc[l], bt, sl, cu, max_q_len=b.max_q_len,
                                     max_kv_len=b.max_kv_len, sinks=self.sinks[l], sum_kv_len=b.sum_kv_len,
                                     seq_lens_host=b.seq_lens, cu_seqlens_q_host=b.cu_seqlens_q)
            ea.o_proj(out, self.wo[l], residual=hidden, out=hidden)
        last = torch.from_numpy(b.cu_seqlens_q[1:].astype("int64") - 1).to(self.dev)
        return self._norm(hidden[last]).float() @ self.emb.float().t()

    # ---- the batching loop -----------------------------------------------------------------
    def _step(self):
        """One shared step over the active requests: prefill chunks within a token budget for
        those still reading their prompt, one decode row for the others."""
        torch = self.torch
        ids, toks, reqs, room = [], [], [], self.step_tokens
        for r in self.active:
            if r.fed < len(r.prompt):
                n = min(self.chunk, len(r.prompt) - r.fed, room)
                if n <= 0:
                    continue              # this step's token budget is spent: next step
                piece = r.prompt[r.fed:r.fed + n]
            else:
                piece, n = [r.last], 1
            room -= n
            ids.append(r.seq_id)
            toks.append(piece)
            reqs.append(r)
        logits = self.forward(ids, toks)
        picks = torch.argmax(logits[:, :EOS + 1], dim=-1).tolist()
        self.steps += 1
        self.mixed_steps += len({len(t) > 1 for t in toks}) == 2
        self.max_step_seqs = max(self.max_step_seqs, len(ids))
        for r, piece, tok in zip(reqs, toks, picks):
            if r.fed < len(r.prompt):
                r.fed += len(piece)
                if r.fed < len(r.prompt):
                    continue              # more prompt to read: nothing sampled yet
            r.last = tok
            r.produced += 1
            r.out.put(tok)                # (EOS included: a genuine stop)
            if tok == EOS or r.produced == r.budget or self.sched.seq_len(r.seq_id) + 1 > self.ctx:
                self._retire(r)

    def _retire(self, r, error=None):
        self.active.remove(r)
        self.committed -= r.blocks
        self.sched.free_seq(r.seq_id)
        r.out.put(error if error is not None else _DONE)

    def _run(self):
        while True:
            with self.cv:
                while not self.waiting and not self.active:
                    self.cv.wait()
                # admission in arrival order, while a slot is free and the pool could hold the
                # request to its last token (a request is never evicted once it runs)
                while (self.waiting and len(self.active) < self.max_seqs
                       and self.committed + self.waiting[0].blocks <= self.num_blocks):
                    r = self.waiting.pop(0)
                    self.sched.add_seq(r.seq_id)
                    self.committed += r.blocks
                    self.active.append(r)
                if not self.active:
                    # nothing runs and the head of the queue cannot be admitted (generate()
                    # refuses requests the pool could never hold, so this is a guard): wait
                    # for the queue to change instead of stepping an empty batch
                    self.cv.wait(timeout=0.05)
                    continue
            try:
                self._step()
            except Exception as e:        # a failed step fails the requests in it, not the process
                for r in list(self.active):
                    self._retire(r, e)

    def generate(self, prompt_ids, max_new_tokens):
        """Greedy decoding through the shared batching loop.  Yields byte tokens, EOS on a
        genuine stop (see FakeEngine.generate)."""
        # The reference asks for min(context_length, 4096) new tokens, i.e. often the whole
        # context (/root/reference/crates/eidola-app-core/src/lib.rs:5595): the budget is cut to
        # what the context can hold behind at least one prompt token, and the prompt keeps its
        # tail (the latest turns) within what is left.
        max_new_tokens = max(1, min(int(max_new_tokens), self.ctx - 1))
        keep = self.ctx - max_new_tokens
        prompt_ids = list(prompt_ids)[-keep:] or [EOS]
        blocks = min((len(prompt_ids) + max_new_tokens + 15) // 16, self.max_blocks)
        if blocks > self.num_blocks:   # could never be admitted: refuse it, do not queue it
            raise RuntimeError(f"request needs {blocks} KV pages, the pool has {self.num_blocks}")
        with self.cv:
            if self.worker is None:
                self.worker = threading.Thread(target=self._run, name="eidola-engine-steps", daemon=True)
                self.worker.start()
            r = _Request(self.next_id, prompt_ids, max_new_tokens)
            self.next_id += 1
            self.waiting.append(r)
            self.cv.notify()
        while True:
            tok = r.out.get()
            if tok is _DONE:
                return
            if isinstance(tok, Exception):
                raise tok
            yield tok


class Handler(BaseHTTPRequestHandler):
    protocol_version = "HTTP/1.1"
    server_version = "eidola-engine-shim/0.1"

    def log_message(self, fmt, *args):   # the supervisor reads stderr only for crashes
        pass

    def _json(self, code, obj):
        body = json.dumps(obj).encode()
        self.send_response(code)
        self.send_header("Content-Type", "application/json")
        self.send_header("Content-Length", str(len(body)))
        self.end_headers()
        self.wfile.write(body)

    def _error(self, code, message, kind="invalid_request_error"):
        self._json(code, {"error": {"message": message, "type": kind, "code": code}})

    def do_GET(self):
        cfg = self.server.cfg
        if self.path == "/health":
            self._json(200, {"status": "ok"})
        elif self.path == "/v1/models":
            self._json(200, {"object": "list", "data": [
                {"id": cfg["alias"], "object": "model", "created": cfg["started"], "owned_by": "eidola_amd"}]})
        else:
            self._error(404, f"no route {self.path}", "not_found")

    def do_POST(self):
        if self.path != "/v1/chat/completions":
            return self._error(404, f"no route {self.path}", "not_found")
        try:
            n = int(self.headers.get("Content-Length", "0"))
            req = json.loads(self.rfile.read(n) or b"{}")
            messages = req["messages"]
            if not isinstance(messages, list) or not messages:
                raise ValueError("messages must be a non-empty list")
            # `tools` (eidola-common/src/lib.rs:129-131) is accepted and not acted upon: the
            # synthetic model cannot call tools, and an engine that ignores the list answers in
            # plain text, which the reference handles.  A malformed list is still a bad request.
            if "tools" in req and not isinstance(req["tools"], list):
                raise ValueError("tools must be a list")
            max_new = int(req.get("max_completion_tokens", req.get("max_tokens", 256)))
            if max_new < 1:
                raise ValueError("max_completion_tokens must be positive")
        except (ValueError, KeyError, TypeError) as e:
            return self._error(400, f"bad request: {e}")
        cfg = self.server.cfg
        model = req.get("model") or cfg["alias"]
        prompt = render_prompt(messages)
        rid, created = "chatcmpl-" + uuid.uuid4().hex[:24], int(time.time())
        gen = cfg["engine"].generate(prompt, max_new)
        if req.get("stream"):
            return self._stream(req, rid, created, model, prompt, gen)
        out, finish = bytearray(), "length"
        try:
            for tok in gen:
                if tok == EOS:
                    finish = "stop"
                    break
                out.append(tok)
        except Exception as e:     # the engine failed this request: say so, keep serving
            return self._error(500, f"engine error: {e}", "server_error")
        self._json(200, {
            "id": rid, "object": "chat.completion", "created": created, "model": model,
            "choices": [{"index": 0, "finish_reason": finish,
                         "message": {"role": "assistant", "content": out.decode("utf-8", "replace")}}],
            "usage": {"prompt_tokens": len(prompt), "completion_tokens": len(out),
                      "total_tokens": len(prompt) + len(out)}})

    def _stream(self, req, rid, created, model, prompt, gen):
        self.send_response(200)
        self.send_header("Content-Type", "text/event-stream")
        self.send_header("Cache-Control", "no-cache")
        self.send_header("Connection", "close")
        self.end_headers()
        self.close_connection = True

        def event(obj):
            self.wfile.write(b"data: " + (obj if isinstance(obj, bytes) else json.dumps(obj).encode()) + b"\n\n")
            self.wfile.flush()

        def chunk(delta, finish=None):
            return {"id": rid, "object": "chat.completion.chunk", "created": created, "model": model,
                    "choices": [{"index": 0, "delta": delta, "finish_reason": finish}]}

        event(chunk({"role": "assistant", "content": ""}))
        n, finish, pending = 0, "length", bytearray()
        try:
            for tok in gen:
                if tok == EOS:
                    finish = "stop"
                    break
                n += 1
                pending.append(tok)
                try:   # only whole UTF-8 sequences go out
                    text = pending.decode("utf-8")
                except UnicodeDecodeError:
                    if len(pending) < 4:
                        continue
                    text = pending.decode("utf-8", "replace")
                pending.clear()
                event(chunk({"content": text}))
        except Exception as e:     # the engine failed mid-stream: an error event, then the usual end
            event({"error": {"message": f"engine error: {e}", "type": "server_error", "code": 500}})
        if pending:
            event(chunk({"content": pending.decode("utf-8", "replace")}))
        event(chunk({}, finish))
        if (req.get("stream_options") or {}).get("include_usage"):
            event({"id": rid, "object": "chat.completion.chunk", "created": created, "model": model, "choices": [],
                   "usage": {"prompt_tokens": len(prompt), "completion_tokens": n, "total_tokens": len(prompt) + n}})
        event(b"[DONE]")


def parse_args(argv=None):
    """The flags the reference passes to its engine, plus the shim's own."""
    ap = argparse.ArgumentParser(prog="eidola-engine-shim", description=__doc__.split("\n\n")[0])
    ap.add_argument("-m", "--model", required=True, help="model file (not read: the model is synthetic)")
    ap.add_argument("--host", default="127.0.0.1")
    ap.add_argument("--port", type=int, default=8080)
    ap.add_argument("--alias", default=None, help="model id reported by /v1/models and echoed in responses")
    ap.add_argument("-c", "--ctx-size", type=int, default=4096)
    ap.add_argument("-ngl", "--n-gpu-layers", type=int, default=999, help="accepted for compatibility")
    ap.add_argument("--jinja", action="store_true", help="accepted for compatibility")
    ap.add_argument("--no-webui", action="store_true", help="accepted for compatibility (there is no web UI)")
    ap.add_argument("--engine", choices=["synthetic", "fake"], default="synthetic")
    ap.add_argument("--layers", type=int, default=4, help="attention blocks of the synthetic model")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("-np", "--parallel", type=int, default=16,
                    help="sequences that may share a step (llama-server's name for its slots)")
    return ap.parse_args(argv)


def make_server(host, port, engine, alias):
    srv = ThreadingHTTPServer((host, port), Handler)
    srv.daemon_threads = True
    srv.cfg = {"engine": engine, "alias": alias, "started": int(time.time())}
    return srv


def main(argv=None):
    a = parse_args(argv)
    engine = FakeEngine() if a.engine == "fake" else SyntheticAttentionEngine(a.layers, a.ctx_size, a.seed,
                                                                             max_seqs=max(1, a.parallel))
    srv = make_server(a.host, a.port, engine, a.alias or a.model)
    try:
        srv.serve_forever()
    except KeyboardInterrupt:
        pass
    finally:
        srv.server_close()


if __name__ == "__main__":
    main()
