#!/usr/bin/env python3
"""Benchmark of the paged sink-attention hot path on one MI355X.

A step = one pass of the hot path over one synthetic batch of BASELINE.json's decode
configuration (configs[1], full-attention variant): the slot-mapped KV write of the 64 new
tokens and split-KV decode attention + merge, all inputs resident in HBM: one
eid_attn_decode call that is handed the new rows (k_new / v_new) and writes them into the
cache itself, or with --unfused eid_kv_write followed by eid_attn_decode.  Page sets rotate
between steps so the 256 MB Infinity Cache cannot serve the KV stream.

Prints ONE JSON line on stdout.  `--all` additionally measures the other configurations
and writes them (one JSON object per line) to the file given by --report.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
# HBM bytes per launch of the dominant kernel on the seeded configs[1] batch, by kernel name,
# from two rocprofv3 --pmc passes over this script (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB; the
# factors are what the same counters read for a plain 1 GiB device copy run with
# --calibrate-copy).  See profiles/splitkv_decode_config2.md.  A kernel that is not listed
# (or a non-default batch) reports traffic as null rather than another kernel's figure.
TRAFFIC_BYTES_PER_LAUNCH = {
    "splitkv_even_kernel<1,bf16,8 waves,direct-to-LDS loads>": int((240_870 * 2.0 + 2_468 * 1.0) * 1024),
}
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
METRIC = "paged sink-attn decode HBM GB/s (% peak) + ragged-batch tokens/s, 1 GPU"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def event_ms(fn, iters, torch):
    """Average milliseconds per call of fn over `iters` back-to-back calls (HIP events on
    torch's current stream, which is the stream every launch here uses)."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(iters):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def split_kernel_ms(w, steps, torch):
    """Average milliseconds of the split-KV launch inside full steps (kv_write, attention),
    from HIP events on the launch stream: one recorded by this script right before the
    attention call, the other by the library right after the split-KV launch
    (args.split_done_event).  The span therefore covers the kernel and the launch gap that
    precedes it, not the merge."""
    pairs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        b.record()  # creates the underlying hipEvent_t
        pairs.append((a, b))
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(pairs):
        if w.fused:
            c = w.fused[i % w.n]
        else:
            w.kv_write(i)
            c = w.attn[i % w.n]
        a.record()
        c.args.split_done_event = b.cuda_event
        c()
    torch.cuda.synchronize()
    for c in w.attn + w.fused:
        c.args.split_done_event = None
    return sum(a.elapsed_time(b) for a, b in pairs) / steps


def kernel_dispatch_ms(calls, steps, torch, n_sets):
    """Average milliseconds of the (last) split-KV / prefill kernel of each call in `calls`
    (PreparedCalls, rotated), from HIP events that the MEASUREMENT build of the library attaches
    to the kernel's own dispatch; None if the calls launch no such kernel."""
    from eidola_amd import _lib
    lib = _lib.load_measure_library()
    bound = [c.bound_to(lib) for c in calls]
    for i in range(2 * n_sets):
        bound[i % n_sets]()
    pairs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    try:
        for i, (a, b) in enumerate(pairs):
            lib.eid_debug_set_kernel_events(a.cuda_event, b.cuda_event)
            bound[i % n_sets]()
    finally:
        lib.eid_debug_set_kernel_events(None, None)
    torch.cuda.synchronize()
    ms = [a.elapsed_time(b) for a, b in pairs]
    return None if min(ms) < 1e-3 else sum(ms) / steps


def split_kernel_dispatch_ms(w, steps, torch, ea):
    """Average milliseconds of the split-KV KERNEL inside full steps: a pair of HIP events per step
    that the MEASUREMENT build of the library (libeidola_attn_measure.so: the same sources with
    -DEID_MEASURE, include/eidola_attn_measure.h) attaches to the kernel's own dispatch
    (hipExtLaunchKernel), so the time between them is the kernel's duration as rocprofv3 reports
    it.  The serving library has no such hook; the steps of this pass run through the
    measurement build, every other figure of the run through the serving library."""
    if not w.fused:
        return None
    from eidola_amd import _lib
    lib = _lib.load_measure_library()
    calls = [c.bound_to(lib) for c in w.fused]
    for i in range(2 * w.n):   # (the second library's first launches: module load, attributes)
        calls[i % w.n]()
    pairs = []
    for _ in range(steps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        b.record()  # creates the underlying hipEvent_t
        pairs.append((a, b))
    torch.cuda.synchronize()
    try:
        for i, (a, b) in enumerate(pairs):
            lib.eid_debug_set_kernel_events(a.cuda_event, b.cuda_event)
            calls[i % w.n]()
    finally:
        lib.eid_debug_set_kernel_events(None, None)
    torch.cuda.synchronize()
    ms = [a.elapsed_time(b) for a, b in pairs]
    if min(ms) < 1e-3:  # (events recorded back to back above: the launch did not take them)
        return None
    return sum(ms) / steps


NO_HINT = False  # --no-hint: do not pass host-side lengths (sum, seq_lens copy) to the library
UNFUSED = False  # --unfused: decode steps as two launches (eid_kv_write, eid_attn_decode)


class Workload:
    """One configuration materialised on the GPU with `nsets` disjoint page sets."""

    def __init__(self, make_batch, nsets, pool_seed, torch, ea, synth, kind, pool=None):
        self.kind = kind  # "decode" or "varlen"
        dev = "cuda:0"
        b0 = make_batch(0)
        nblk = int(((b0.seq_lens.astype("int64") + 15) // 16).sum())
        self.batches = [b0] + [make_batch(r * nblk) for r in range(1, nsets)]
        g = b0.geom
        self.geom = g
        if pool is not None:   # another workload's pool of the same dtype and size
            self.k_cache, self.v_cache, self.k_scale, self.v_scale = pool
            assert self.k_cache.shape[0] == b0.num_blocks
        else:
            dt = torch.uint8 if g.kv_dtype == ea.KV_FP8_E4M3 else torch.bfloat16
            self.k_cache = torch.empty((b0.num_blocks, 16, g.num_kv_heads, 64), dtype=dt, device=dev)
            self.v_cache = torch.empty_like(self.k_cache)
            t0 = time.time()
            self.k_scale, self.v_scale = synth.fill_pool_gpu(g, self.k_cache, self.v_cache, pool_seed)
            torch.cuda.synchronize()
            log(f"[bench] {b0.name}: pool of {b0.num_blocks} blocks filled in {time.time()-t0:.1f}s, "
                f"{nsets} page sets of {nblk} blocks")
        self.pool = (self.k_cache, self.v_cache, self.k_scale, self.v_scale)
        T = b0.num_q_tokens

        def bf16(bits):
            import numpy as np
            return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.bfloat16)

        self.q = bf16(synth.normal_bf16((T, g.num_q_heads, 64), b0.seed, synth.TID_Q))
        self.k_new = bf16(synth.normal_bf16((T, g.num_kv_heads, 64), b0.seed, synth.TID_K))
        self.v_new = bf16(synth.normal_bf16((T, g.num_kv_heads, 64), b0.seed, synth.TID_V))
        self.sinks = torch.from_numpy(synth.bf16_bits_to_f32(
            synth.normal_bf16((g.num_q_heads,), b0.seed, synth.TID_SINK))).to(dev)
        self.seq_lens = torch.from_numpy(b0.seq_lens).to(dev)
        self.cu = torch.from_numpy(b0.cu_seqlens_q).to(dev)
        self.slots = [torch.from_numpy(b.slot_mapping).to(dev) for b in self.batches]
        self.tables = [torch.from_numpy(b.block_table).to(dev) for b in self.batches]
        fn = "eid_attn_decode" if kind == "decode" else "eid_attn_varlen"
        ws = None
        self.attn, self.merge, self.fused = [], [], []
        for bt in self.tables:
            # the scheduler builds seq_lens / cu_seqlens_q on the host: the library gets those
            # copies (and their sum) and plans the launches with them
            kw = dict(max_q_len=b0.max_q_len, max_kv_len=b0.max_kv_len, sinks=self.sinks,
                      k_scale=self.k_scale, v_scale=self.v_scale, workspace=ws,
                      sum_kv_len=0 if NO_HINT else int(b0.seq_lens.sum()),
                      seq_lens_host=None if NO_HINT else b0.seq_lens,
                      cu_seqlens_q_host=None if NO_HINT or kind != "varlen" else b0.cu_seqlens_q)
            if kind == "decode" and not NO_HINT:
                kw["block_table_host"] = bt.cpu().numpy()
            cu = self.cu if kind == "varlen" else None
            c = ea.prepare(fn, g, self.q, self.k_cache, self.v_cache, bt, self.seq_lens, cu, **kw)
            ws = c._keep[-1]
            self.attn.append(c)
            kw["workspace"] = ws
            if kind == "decode" and not UNFUSED:
                # the decode step as ONE call: the newest token's KV rows go in with the call,
                # which writes them into the cache itself (stage K1 fused into K2)
                self.fused.append(ea.prepare(fn, g, self.q, self.k_cache, self.v_cache, bt,
                                             self.seq_lens, None, k_new=self.k_new,
                                             v_new=self.v_new, **kw))
            self.merge.append(ea.prepare("eid_lse_merge", g, self.q, self.k_cache, self.v_cache,
                                         bt, self.seq_lens, cu, **kw))
        self.ea = ea
        self.n = nsets

    def kv_write(self, i):
        self.ea.kv_write(self.geom, self.k_new, self.v_new, self.k_cache, self.v_cache,
                         self.slots[i % self.n], self.k_scale, self.v_scale)

    def step(self, i):
        """One pass of the hot path over one batch: KV write of the new tokens, attention."""
        if self.fused:
            self.fused[i % self.n]()
        else:
            self.step_unfused(i)

    def step_unfused(self, i):
        self.kv_write(i)
        self.attn[i % self.n]()


def graph_step_ms(w, steps, torch):
    """The same steps replayed from a HIP graph: all page sets' steps (kv_write + attention)
    are captured once on a side stream and the graph is replayed, which removes the host's
    launch cost from short steps.  Returns milliseconds per step, or None if capture fails."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(w.n):
                w.step(i)                      # warm-up on the capture stream
            side.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for i in range(w.n):
                    w.step(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        reps = max(1, steps // w.n)
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * w.n)
    except Exception as ex:  # capture is an extra; the eager numbers stand without it
        log(f"[bench] graph capture unavailable: {ex}")
        return None


def measure(w, steps, warmup, torch, synth, label):
    b = w.batches[0]
    for i in range(warmup):
        w.step(i)
    ms_step = event_ms(w.step, steps, torch)
    ms_unfused = event_ms(w.step_unfused, steps, torch) if w.fused else ms_step
    ms_attn = event_ms(lambda i: w.attn[i % w.n](), steps, torch)
    ms_merge = event_ms(lambda i: w.merge[i % w.n](), steps, torch)
    ms_write = event_ms(w.kv_write, steps, torch)
    ms_split = split_kernel_ms(w, steps, torch)
    ms_graph = graph_step_ms(w, steps, torch)
    work = synth.algorithmic_work(b)
    work_w = synth.algorithmic_work(b, include_kv_write=True)
    r = {
        "config": label, "ms_per_step": ms_step, "ms_per_step_two_launches": ms_unfused,
        "fused_kv_write": bool(w.fused), "ms_attn": ms_attn, "ms_merge": ms_merge,
        "ms_kv_write": ms_write, "ms_split": ms_split, "ms_per_step_graph": ms_graph, "alg_bytes": work["bytes"], "alg_flops": work["flops"],
        "q_tokens": work["q_tokens"], "ctx_tokens": work["ctx_tokens"],
        "step_GBps": work_w["bytes"] / ms_step / 1e6,
        "attn_GBps": work["bytes"] / ms_attn / 1e6,
        "attn_TFLOPs": work["flops"] / ms_attn / 1e9,
        "q_tokens_per_s": work["q_tokens"] / ms_step * 1e3,
        "ctx_tokens_per_s": work["ctx_tokens"] / ms_step * 1e3,
    }
    # the split-KV launch records the partition it ran with at the head of the workspace
    # (meaningless when no sequence of the first class ran: reported as None)
    part = int(w.attn[0]._keep[-1][:4].view(torch.int32).item())
    r["partition"] = part if 64 <= part <= 4096 and part % 64 == 0 else None
    gtxt = f", graph replay {ms_graph*1e3:.1f}" if ms_graph else ""
    if w.fused:
        gtxt += f", as kv_write + attention {ms_unfused*1e3:.1f}"
    log(f"[bench] {label}: step {ms_step*1e3:.1f} us{gtxt} (attn {ms_attn*1e3:.1f}, split-KV "
        f"{ms_split*1e3:.1f}, merge {ms_merge*1e3:.1f}, kv_write {ms_write*1e3:.1f}); attn {r['attn_GBps']:.0f} GB/s = "
        f"{100*r['attn_GBps']/HBM_PEAK_GBS:.1f}% HBM, {r['attn_TFLOPs']:.1f} TFLOP/s; "
        f"partition {r['partition']}")
    return r


def subset(batch, idx, name, synth):
    """The sequences `idx` of a batch as a batch of their own (same pages, same geometry)."""
    import numpy as np
    idx = np.asarray(idx)
    return synth.Batch(name, batch.geom, batch.seq_lens[idx], batch.q_lens[idx],
                       batch.block_table[idx], batch.num_blocks, batch.seed)


def compact_pass(w, steps, warmup, torch):
    """(ms per step, ms per attention call) of a workload: HIP events around `steps`
    back-to-back steps / calls, page sets rotated."""
    for i in range(warmup):
        w.step(i)
    # The core clock settles over the first ~20 ms of a new kind of load (an MFMA-bound kernel
    # that follows memory-bound ones runs ~10 % slower until then): warm up for that long
    # and time at least 10 ms of work.
    est = max(event_ms(w.step, 5, torch), 1e-3)
    for i in range(int(20.0 / est) + 1):
        w.step(i)
    n = max(steps, int(10.0 / est) + 1)
    ms_step = event_ms(w.step, n, torch)
    ms_attn = event_ms(lambda i: w.attn[i % w.n](), n, torch)
    return ms_step, ms_attn


def parity_sample(w, seqs, torch, synth, what):
    """Checker of the cpu_baseline leg: the attention output of page set 0 for the sequences
    `seqs` against the CPU restatement's fp64 path on a compacted copy of their pages;
    returns (max abs, mean abs) error."""
    import numpy as np
    import oracle
    import eidola_amd as ea
    b = w.batches[0]
    seqs = [int(x) for x in seqs]
    nblk = (b.seq_lens[seqs].astype(np.int64) + 15) // 16
    pages = np.concatenate([b.block_table[s, :n] for s, n in zip(seqs, nblk)])
    idx = torch.from_numpy(pages.astype(np.int64)).to("cuda:0")

    def host(t):
        t = t[idx].cpu().contiguous()
        return t.numpy() if t.dtype == torch.uint8 else t.view(torch.int16).numpy().view(np.uint16)

    kc, vc = host(w.k_cache), host(w.v_cache)
    bt = np.zeros((len(seqs), int(nblk.max())), np.int32)
    off = 0
    for i, n in enumerate(nblk):
        bt[i, :n] = np.arange(off, off + n)
        off += int(n)
    sub = synth.Batch(b.name + "_sample", b.geom, b.seq_lens[seqs], b.q_lens[seqs], bt, len(pages), b.seed)
    d = ea.make_desc(sub.geom, num_seqs=sub.num_seqs, num_q_tokens=sub.num_q_tokens,
                     max_q_len=sub.max_q_len, max_kv_len=sub.max_kv_len,
                     max_blocks_per_seq=bt.shape[1], num_blocks=len(pages))
    cu = b.cu_seqlens_q
    rows = np.concatenate([np.arange(cu[s], cu[s + 1]) for s in seqs])
    q = w.q.cpu().view(torch.int16).numpy().view(np.uint16)[rows]
    ks = w.k_scale.cpu().numpy() if w.k_scale is not None else None
    vs = w.v_scale.cpu().numpy() if w.v_scale is not None else None
    ref, _ = oracle.attn_f64(d, q, kc, vc, bt, sub.seq_lens, sub.cu_seqlens_q, w.sinks.cpu().numpy(), ks, vs)
    out = w.attn[0]()
    torch.cuda.synchronize()
    got = synth.bf16_bits_to_f32(out.cpu().view(torch.int16).numpy().view(np.uint16)[rows]).astype(np.float64)
    err = np.abs(got - ref)
    log(f"[bench] {what}: {len(seqs)} sampled sequences ({len(rows)} rows) vs the fp64 CPU restatement: "
        f"max abs {err.max():.2e}, mean abs {err.mean():.2e}")
    return {"max_abs": float(err.max()), "mean_abs": float(err.mean()), "rows": int(len(rows)),
            "sequences": seqs}


def other_configs(a, torch, ea, synth, pool2, check):
    """Compact passes over the other BASELINE configurations: per (config, variant) the time of
    the attention call, the algorithmic work and the roofline fraction it gives; with `check`,
    sampled sequences against the CPU restatement (part of the cpu_baseline leg)."""
    import numpy as np
    steps, warm = max(10, a.steps // 8), max(3, a.warmup // 4)
    out = {}

    def hbm(work, ms, kernel, extra=None, kernel_ms=None):
        """`frac` is quoted on the whole CALL (every launch of it, merge included); frac_kernel on
        the dominant kernel alone (events on its own dispatch, measurement build)."""
        gbs = work["bytes"] / ms / 1e6
        r = {"ms_call": ms, "call_us": ms * 1e3, "kernel_us": kernel_ms * 1e3 if kernel_ms else None,
             "alg_bytes": work["bytes"], "q_tokens": work["q_tokens"],
             "roofline": {"bound": "hbm", "kernel": kernel, "achieved": gbs, "peak": HBM_PEAK_GBS,
                          "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "frac_uses": "call_us",
                          "frac_kernel": (work["bytes"] / kernel_ms / 1e6 / HBM_PEAK_GBS) if kernel_ms else None,
                          "how": "call_us: HIP events around back-to-back eid_attn_* calls (every launch of the "
                                 "call), page sets rotated; kernel_us: events attached to the dominant "
                                 "kernel's dispatch by the measurement build of the library"}}
        r.update(extra or {})
        return r

    kdur = lambda w_, n: kernel_dispatch_ms(w_.attn, n, torch, w_.n)

    # ---- 2b: decode, 128-token window (latency-bound: 17 MB of KV) ----
    w = Workload(lambda off: synth.config2(window=128, perm_offset=off), a.sets, 7, torch, ea, synth,
                 "decode", pool=pool2)
    ms_step, ms_attn = compact_pass(w, steps * 2, warm, torch)
    out["2b_window"] = hbm(synth.algorithmic_work(w.batches[0]), ms_attn, "shortspan_kernel<1,bf16>",
                           {"ms_per_step": ms_step, "tokens_per_s": 64 / ms_step * 1e3,
                            "note": "latency-bound: 17 MB of KV per call; one launch (kernel = call)"})
    if check:
        order = np.argsort(w.batches[0].seq_lens)
        out["2b_window"]["parity"] = parity_sample(w, [order[0], order[31], order[-1], 0, 1], torch, synth, "2b_window")
    # ---- 3: mixed chunked prefill + decode; the two populations also on their own ----
    full = lambda off: synth.config3(perm_offset=off)
    w3 = Workload(full, 4, 8, torch, ea, synth, "varlen", pool=pool2)
    ms_step, ms_attn = compact_pass(w3, steps, warm, torch)
    b3 = w3.batches[0]
    lw, sw = synth.algorithmic_work(b3, rows="long"), synth.algorithmic_work(b3, rows="short")
    out["3_mixed"] = {"ms_call": ms_attn, "call_us": ms_attn * 1e3, "kernel_us": None,
                      "ms_per_step": ms_step, "q_tokens": b3.num_q_tokens,
                      "tokens_per_s": b3.num_q_tokens / ms_step * 1e3,
                      "prefill_TFLOPs_of_the_call": lw["flops"] / ms_attn / 1e9,
                      "decode_GBps_of_the_call": sw["bytes"] / ms_attn / 1e6,
                      "note": "two streams: the split-KV rows take every second CU, the prefill "
                              "workgroups the others and then the rest"}
    if check:
        lens8 = np.argsort(b3.seq_lens[:8])
        out["3_mixed"]["parity"] = parity_sample(w3, [lens8[0], lens8[-1], 8, 9, 60, 127], torch, synth, "3_mixed")
    wp = Workload(lambda off: subset(full(off), np.arange(8), "config3_prefill_rows", synth), 4, 8,
                  torch, ea, synth, "varlen", pool=pool2)
    _, ms_p = compact_pass(wp, steps, warm, torch)
    ms_pk = kdur(wp, steps)
    tf = lw["flops"] / ms_p / 1e9
    out["3_prefill"] = {"ms_call": ms_p, "call_us": ms_p * 1e3, "kernel_us": ms_pk * 1e3 if ms_pk else None,
                        "alg_flops": lw["flops"], "q_tokens": lw["q_tokens"],
                        "roofline": {"bound": "mfma", "kernel": "prefill_kernel<bf16, folded softmax factor>",
                                     "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": tf / MFMA_BF16_PEAK_TFLOPS, "frac_uses": "call_us",
                                     "frac_kernel": (lw["flops"] / ms_pk / 1e9 / MFMA_BF16_PEAK_TFLOPS) if ms_pk else None,
                                     "how": "call_us: HIP events around back-to-back eid_attn_varlen calls on "
                                            "the 8 prefill sequences alone (one launch); kernel_us: events on "
                                            "the kernel's dispatch (measurement build)"}}
    if check:
        out["3_prefill"]["parity"] = parity_sample(wp, [0, 3, 7], torch, synth, "3_prefill")
    wd = Workload(lambda off: subset(full(off), np.arange(8, 128), "config3_decode_rows", synth), 4, 8,
                  torch, ea, synth, "varlen", pool=pool2)
    _, ms_d = compact_pass(wd, steps, warm, torch)
    out["3_decode"] = hbm(sw, ms_d, "splitkv_even_kernel<1,bf16,8 waves,direct-to-LDS loads>", kernel_ms=kdur(wd, steps))
    if check:
        order = np.argsort(wd.batches[0].seq_lens)
        out["3_decode"]["parity"] = parity_sample(wd, [order[0], order[30], order[60], order[90], order[-1]], torch,
                                                  synth, "3_decode")
    w = w3 = wp = wd = None
    # ---- 4: fp8 KV decode ----
    w4 = Workload(lambda off: synth.config4(num_blocks=300_000, perm_offset=off), 3, 9, torch, ea,
                  synth, "decode")
    ms_step, ms_attn = compact_pass(w4, steps, warm, torch)
    out["4_fp8"] = hbm(synth.algorithmic_work(w4.batches[0]), ms_attn,
                       "splitkv_even_kernel<1,fp8,4 waves,head pairs,direct-to-LDS loads>",
                       {"ms_per_step": ms_step, "tokens_per_s": 256 / ms_step * 1e3}, kernel_ms=kdur(w4, steps))
    if check:
        order = np.argsort(w4.batches[0].seq_lens)
        out["4_fp8"]["parity"] = parity_sample(w4, [order[0], order[127], order[-1], 0, 1], torch, synth, "4_fp8")
    w4 = None
    torch.cuda.empty_cache()
    # ---- 5: speculative verify, 512-token partitions; layer 0 full, layer 1 windowed ----
    pool5, t5 = None, 0.0
    for layer, key in ((0, "5_full"), (1, "5_window")):
        w5 = Workload(lambda off: synth.config5(layer=layer, num_blocks=900_000, perm_offset=off), 3,
                      10, torch, ea, synth, "varlen", pool=pool5)
        pool5 = w5.pool
        ms_step, ms_attn = compact_pass(w5, max(5, steps // 2), warm, torch)
        t5 += ms_step
        n5 = max(5, steps // 2)
        out[key] = hbm(synth.algorithmic_work(w5.batches[0]), ms_attn,
                       "splitkv_even_kernel<3,bf16,8 waves,direct-to-LDS loads>" if layer == 0
                       else "splitkv_kernel<3,bf16,8 waves,direct-to-LDS loads>, one item per sequence",
                       {"ms_per_step": ms_step, "partition_size": 512}, kernel_ms=kdur(w5, n5))
        if layer == 0:
            out[key]["partials"] = ("ranges cut on the 512-key grid, one workgroup per range; the consecutive "
                                    "partitions a workgroup holds of one sequence are merged in registers and "
                                    "stored as one partial; what crosses workgroups goes through the merge kernel")
            # the same batch with every 512-key partition stored and merged by the merge kernel
            # (a switch of the measurement build; the calls of this pass run through that build)
            from eidola_amd import _lib
            mlib = _lib.load_measure_library()
            bound = [c.bound_to(mlib) for c in w5.attn]
            mlib.eid_debug_set_store_every_partition(1)
            try:
                for i in range(2 * w5.n):
                    bound[i % w5.n]()
                ms_every = event_ms(lambda i: bound[i % w5.n](), n5, torch)
                ms_every_k = kernel_dispatch_ms(w5.attn, n5, torch, w5.n)
            finally:
                mlib.eid_debug_set_store_every_partition(-1)
            out["5_full_every_partition_stored"] = hbm(
                synth.algorithmic_work(w5.batches[0]), ms_every,
                "splitkv_even_kernel<3,bf16,8 waves,direct-to-LDS loads>, a partial per 512-key partition",
                {"partition_size": 512,
                 "partials": "every 512-key partition stored (346 MB of partials) and merged by the merge kernel"},
                kernel_ms=ms_every_k)
        if check:
            order = np.argsort(w5.batches[0].seq_lens)
            out[key]["parity"] = parity_sample(w5, [order[0], order[64], order[-1]], torch, synth, key)
        w5 = None
    out["5_full"]["tokens_per_s_both_layers"] = 640 / t5 * 1e3
    for k, v in out.items():
        rf = v.get("roofline")
        if rf:
            log(f"[bench] {k}: call {v['ms_call']*1e3:.1f} us, {rf['achieved']:.0f} {rf['unit']} = "
                f"{100*rf['frac']:.1f}% of the {rf['bound']} peak")
        else:
            log(f"[bench] {k}: call {v['ms_call']*1e3:.1f} us, step {v['ms_per_step']*1e3:.1f} us")
    return out


def sched_bench(synth, ea, steps=200):
    """Host cost of the batch-metadata builder on the decode configuration: 64 sequences
    with config 2's context lengths are prefilled through the scheduler, then `steps`
    decode steps (one new token per sequence) are built; microseconds per built step."""
    import numpy as np
    b = synth.config2()
    mb = b.block_table.shape[1] + (steps + 15) // 16 + 1   # room for the decode steps
    sched = ea.Scheduler(b.num_blocks, mb, prefix_reuse=True)
    ids = np.arange(b.num_seqs, dtype=np.int64)
    for i in ids:
        sched.add_seq(int(i))
    rng = np.random.default_rng(1)
    first = np.maximum(b.seq_lens - 1, 1).astype(np.int32)
    t0 = time.perf_counter()
    sched.build_batch(ids, first, rng.integers(0, 50000, size=int(first.sum())))
    t_prefill = time.perf_counter() - t0
    ones = np.ones(b.num_seqs, dtype=np.int32)
    # calling through the raw ABI with preallocated buffers, as an engine loop would
    import ctypes as C
    from eidola_amd._lib import BatchInfo
    lib = ea.load_library()
    bt = np.zeros((b.num_seqs, mb), np.int32)
    slot, cu = np.empty(b.num_seqs, np.int64), np.empty(b.num_seqs + 1, np.int32)
    sl, pos, tok = np.empty(b.num_seqs, np.int32), np.empty(b.num_seqs, np.int32), np.zeros(b.num_seqs, np.int32)
    info = BatchInfo()
    t0 = time.perf_counter()
    for _ in range(steps):
        rc = lib.eid_sched_build_batch(sched._h, ids.ctypes.data, ones.ctypes.data, b.num_seqs,
                                       tok.ctypes.data, bt.ctypes.data, slot.ctypes.data,
                                       cu.ctypes.data, sl.ctypes.data, pos.ctypes.data, C.byref(info))
        assert rc == 0
    us = (time.perf_counter() - t0) / steps * 1e6
    r = {"config": "sched_build_batch_decode64", "host_us_per_step": us,
         "prefill_build_ms": t_prefill * 1e3, "prefill_tokens": int(first.sum()),
         "sum_kv_len": int(info.sum_kv_len)}
    log(f"[bench] scheduler: {us:.1f} us of host time per 64-sequence decode step "
        f"(prefix index on); building the {int(first.sum())}-token prefill batch took "
        f"{t_prefill*1e3:.1f} ms")
    return r


def rope_bench(torch, ea, synth, steps=50):
    """eid_rope_kv_write on config 3's new tokens (4,216) and on a 64-token decode step:
    HBM-bound; algorithmic bytes = T * (qkv row read 10,240 + q row written 8,192 + k and v
    rows written 2 * 1,024) + the cos/sin rows read."""
    import numpy as np
    g = ea.AttnGeometry()
    nb = 20000
    kc = torch.zeros((nb, 16, 8, 64), dtype=torch.bfloat16, device="cuda:0")
    vc = torch.zeros_like(kc)
    table = torch.from_numpy(ea.yarn_cos_sin(8192)).to("cuda:0")
    out = []
    for T in (4216, 64):
        qkv = torch.randn((T, 5120), device="cuda:0").to(torch.bfloat16)
        pos = torch.randint(0, 8192, (T,), dtype=torch.int32, device="cuda:0")
        slots = torch.randperm(nb * 16, device="cuda:0")[:T].to(torch.int64)
        q = torch.empty((T, 64, 64), dtype=torch.bfloat16, device="cuda:0")
        fn = lambda i: ea.rope_kv_write(g, qkv, pos, table, kc, vc, slots, q_out=q)
        for i in range(5):
            fn(i)
        ms = event_ms(fn, steps, torch)
        nbytes = T * (10240 + 8192 + 2048 + 256)
        r = {"config": f"rope_kv_write_{T}_tokens", "ms": ms, "alg_bytes": nbytes,
             "GBps": nbytes / ms / 1e6}
        log(f"[bench] rope_kv_write, {T} tokens: {ms*1e3:.1f} us per call, "
            f"{r['GBps']:.0f} GB/s = {100*r['GBps']/HBM_PEAK_GBS:.1f}% HBM")
        out.append(r)
    return out


def oproj_bench(torch, ea):
    """eid_o_proj on gpt-oss's shape (4096 -> 2880, bias + residual) for a 64-token decode
    step, batches of 256, 512 and 1,024 tokens and config 3's 4,216 tokens.  16 weight copies (377 MB, more than
    the last-level cache) are used in turn, as the layers of a model would be; 16 launches
    are captured in a HIP graph and its replay timed with events, so the figure is device
    time, not Python call overhead.  Up to 64 tokens the kernel is HBM-bound (algorithmic
    bytes = weight + activations in + residual in + out), beyond that MFMA-bound
    (2 T N K flops).  torch.addmm (hipBLASLt) on the same buffers is timed beside it."""
    N, K, L = 2880, 4096, 16
    ws = [torch.randn(N, K, device="cuda:0").to(torch.bfloat16) * 0.02 for _ in range(L)]
    bias = torch.randn(N, device="cuda:0").to(torch.bfloat16)
    out = []
    for T in (64, 256, 512, 1024, 4216):
        x = torch.randn(T, K, device="cuda:0").to(torch.bfloat16)
        res = torch.randn(T, N, device="cuda:0").to(torch.bfloat16)
        y = torch.empty(T, N, dtype=torch.bfloat16, device="cuda:0")
        fns = {"eid": lambda i: ea.o_proj(x, ws[i], bias, res, out=y),
               "hipblaslt": lambda i: torch.addmm(res, x, ws[i].t(), out=y)}
        r = {"config": f"o_proj_{T}_tokens", "flops": 2.0 * T * N * K,
             "alg_bytes": 2 * (N * K + T * K + 2 * T * N + N)}
        for name, fn in fns.items():
            for i in range(2):
                fn(i)
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                fn(0)
                torch.cuda.synchronize()
                with torch.cuda.graph(graph, stream=side):
                    for i in range(L):
                        fn(i)
            torch.cuda.synchronize()
            graph.replay()
            ms = event_ms(lambda i: graph.replay(), 5, torch) / L
            r[name + "_ms"] = ms
        r["GBps"] = r["alg_bytes"] / r["eid_ms"] / 1e6
        r["TFLOPs"] = r["flops"] / r["eid_ms"] / 1e9
        log(f"[bench] o_proj, {T} tokens: {r['eid_ms']*1e3:.1f} us per call "
            f"({r['GBps']:.0f} GB/s = {100*r['GBps']/HBM_PEAK_GBS:.1f}% HBM, "
            f"{r['TFLOPs']:.0f} TFLOP/s = {100*r['TFLOPs']/2500:.1f}% of bf16 MFMA peak); "
            f"hipBLASLt {r['hipblaslt_ms']*1e3:.1f} us")
        out.append(r)
    return out


def prefill_bench(torch, ea, synth):
    """Chunked prefill of ONE long prompt: a 512-token and a 2,048-token chunk behind 60,000
    tokens of context (few query tiles, so the prefill kernel splits every tile's key range),
    and an 8,192-token chunk without prior.  MFMA-bound: 16,384 FLOP per unmasked pair."""
    import numpy as np
    g = ea.AttnGeometry()
    nb = 300_000
    kc = torch.empty((nb, 16, 8, 64), dtype=torch.bfloat16, device="cuda:0")
    vc = torch.empty_like(kc)
    synth.fill_pool_gpu(g, kc, vc, 12)
    sinks = torch.zeros(64, device="cuda:0")
    out = []
    for new, prior in ((512, 60_000), (2048, 60_000), (8192, 0)):
        lens = np.array([new + prior], np.int32)
        q = torch.randn((new, 64, 64), device="cuda:0").to(torch.bfloat16)
        bt = torch.from_numpy(synth.build_block_table(lens, nb, 12)).to("cuda:0")
        call = ea.prepare("eid_attn_varlen", g, q, kc, vc, bt, torch.from_numpy(lens).to("cuda:0"),
                          torch.tensor([0, new], dtype=torch.int32, device="cuda:0"),
                          max_q_len=new, max_kv_len=new + prior, sinks=sinks,
                          sum_kv_len=new + prior)
        for _ in range(3):
            call()
        ms = event_ms(lambda i: call(), 10, torch)
        flops = 16384.0 * (new * prior + new * (new + 1) // 2)
        r = {"config": f"prefill_{new}_new_after_{prior}", "ms": ms, "flops": flops,
             "TFLOPs": flops / ms / 1e9}
        log(f"[bench] prefill, {new} new tokens after {prior}: {ms*1e3:.1f} us, "
            f"{r['TFLOPs']:.0f} TFLOP/s = {100*r['TFLOPs']/MFMA_BF16_PEAK_TFLOPS:.1f}% of bf16 MFMA peak")
        out.append(r)
    return out


def small_batch_bench(torch, ea, synth):
    """Decode steps of small batches (one to sixteen sequences), the latency regime: replayed
    from a HIP graph over several page sets, KV write fused.  The figure is microseconds per
    call; the bandwidth column only says how far from streaming the call is."""
    import numpy as np
    g = ea.AttnGeometry()
    nb = 300_000
    kc = torch.empty((nb, 16, 8, 64), dtype=torch.bfloat16, device="cuda:0")
    vc = torch.empty_like(kc)
    synth.fill_pool_gpu(g, kc, vc, 13)
    sinks = torch.zeros(64, device="cuda:0")
    out = []
    for lens in ([512], [4096], [16384], [131072], [8192] * 4, [2048] * 16,
                 [8000, 4000, 2000, 1000, 500, 250, 125, 64]):
        lens = np.array(lens, np.int32)
        B, total = len(lens), int(lens.sum())
        q = torch.randn((B, 64, 64), device="cuda:0").to(torch.bfloat16)
        kn = torch.randn((B, 8, 64), device="cuda:0").to(torch.bfloat16)
        vn = torch.randn((B, 8, 64), device="cuda:0").to(torch.bfloat16)
        sl = torch.from_numpy(lens).to("cuda:0")
        nblk = int(((lens.astype(np.int64) + 15) // 16).sum())
        nsets = max(1, min(8, nb // nblk))
        calls, ws = [], None
        for r in range(nsets):
            bt = torch.from_numpy(synth.build_block_table(lens, nb, 13, perm_offset=r * nblk)).to("cuda:0")
            c = ea.prepare("eid_attn_decode", g, q, kc, vc, bt, sl, None, max_kv_len=int(lens.max()),
                           sinks=sinks, sum_kv_len=total, seq_lens_host=lens, workspace=ws,
                           k_new=kn, v_new=vn)
            ws = c._keep[-1]
            calls.append(c)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for c in calls:
                c(stream=side.cuda_stream)
            side.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=side):
                for _ in range(4):
                    for c in calls:
                        c(stream=side.cuda_stream)
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        us = event_ms(lambda i: gr.replay(), 5, torch) * 1e3 / (4 * nsets)
        name = f"{B}x{int(lens.max())}" + ("" if lens.min() == lens.max() else "_ragged")
        r = {"config": f"small_batch_decode_{name}", "us": us, "bytes": total * 2048,
             "partition": ea.partition_size(calls[0].desc)}
        log(f"[bench] small batch {name}: {us:.1f} us per decode call "
            f"({total * 2048 / us / 1e3:.0f} GB/s); partition {r['partition']}")
        out.append(r)
    return out


def stack_bench(torch, ea, synth, layers=36, fused_qkv=True):
    """The attention block of every layer of ONE decode step, replayed from one HIP graph:
    per layer the QKV projection (the library's GEMM entry point, 2880 -> 5120 with bias),
    rotary embedding + split + KV write, paged sink-attention (even layers a 128-token
    window, odd layers full attention, as gpt-oss alternates) and the output projection with
    bias and residual add (4096 -> 2880).  Config 2's batch (64 sequences); every layer has
    its own pages (one pool, disjoint page sets) and its own weights, so nothing is served
    from a cache that a real model would not have.  Norms, MoE and sampling are not here."""
    import numpy as np
    dev = "cuda:0"
    b0 = synth.config2()
    S, H, NQKV = b0.num_seqs, 2880, (64 + 2 * 8) * 64
    nblk = int(((b0.seq_lens.astype(np.int64) + 15) // 16).sum())
    nb = layers * nblk
    gfull, gwin = ea.AttnGeometry(), ea.AttnGeometry(window=128)
    kc = torch.empty((nb, 16, 8, 64), dtype=torch.bfloat16, device=dev)
    vc = torch.empty_like(kc)
    synth.fill_pool_gpu(gfull, kc, vc, 21)
    sl_h = b0.seq_lens
    sl = torch.from_numpy(sl_h).to(dev)
    pos = torch.from_numpy((sl_h - 1).astype(np.int32)).to(dev)
    cos_sin = torch.from_numpy(ea.yarn_cos_sin(int(sl_h.max()) + 1)).to(dev)
    sinks = torch.zeros(64, device=dev)
    hidden0 = (torch.randn((S, H), device=dev) * 0.5).to(torch.bfloat16)
    hidden = hidden0.clone()
    qkv = torch.empty((S, NQKV), dtype=torch.bfloat16, device=dev)
    q = torch.empty((S, 64, 64), dtype=torch.bfloat16, device=dev)
    lay, ws = [], {}
    for l in range(layers):
        batch = synth.config2(num_blocks=nb, perm_offset=l * nblk)
        bt = torch.from_numpy(batch.block_table).to(dev)
        g = gwin if l % 2 == 0 else gfull
        call = ea.prepare("eid_attn_decode", g, q, kc, vc, bt, sl, None, max_kv_len=b0.max_kv_len,
                          sinks=sinks, sum_kv_len=int(sl_h.sum()), seq_lens_host=sl_h,
                          workspace=ws.get(l % 2))
        ws[l % 2] = call._keep[-1]
        lay.append(dict(
            wqkv=(torch.randn((NQKV, H), device=dev) * 0.02).to(torch.bfloat16),
            bqkv=torch.zeros(NQKV, dtype=torch.bfloat16, device=dev),
            wo=(torch.randn((H, 4096), device=dev) * 0.02).to(torch.bfloat16),
            bo=torch.zeros(H, dtype=torch.bfloat16, device=dev),
            slots=torch.from_numpy(batch.slot_mapping).to(dev), geom=g, attn=call))

    def step(stream=None):
        hidden.copy_(hidden0)
        for L in lay:
            if fused_qkv:
                ea.qkv_rope_kv_write(L["geom"], hidden, L["wqkv"], L["bqkv"], pos, cos_sin, kc, vc,
                                     L["slots"], q_out=q)
            else:
                ea.o_proj(hidden, L["wqkv"], L["bqkv"], out=qkv)
                ea.rope_kv_write(L["geom"], qkv, pos, cos_sin, kc, vc, L["slots"], q_out=q)
            L["attn"](stream=stream)
            ea.o_proj(L["attn"].out, L["wo"], L["bo"], residual=hidden, out=hidden)

    step()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(side.cuda_stream)
        side.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=side):
            step(side.cuda_stream)
    torch.cuda.synchronize()
    gr.replay()
    torch.cuda.synchronize()
    ms = event_ms(lambda i: gr.replay(), 20, torch)
    ms_eager = event_ms(lambda i: step(), 5, torch)
    ok = bool(torch.isfinite(hidden.float()).all().item())
    kv_bytes = sum(synth.algorithmic_work(synth.config2(window=0 if l % 2 else 128))["bytes"]
                   for l in range(layers))
    w_bytes = layers * (NQKV * H + H * 4096) * 2
    r = {"config": f"attention_stack_{layers}_layers_config2_batch" + ("" if fused_qkv else "_qkv_unfused"),
         "ms": ms, "ms_eager": ms_eager,
         "layers": layers, "us_per_layer": ms * 1e3 / layers, "kv_bytes": kv_bytes,
         "weight_bytes": w_bytes, "GBps": (kv_bytes + w_bytes) / ms / 1e6, "finite": ok}
    log(f"[bench] attention stack, {layers} layers x ("
        + ("QKV proj + RoPE + KV write in one launch" if fused_qkv else "QKV proj, RoPE + KV write")
        + f", attention, o_proj), 64 seqs: {ms*1e3:.0f} us per decode step from one graph "
        f"({ms*1e3/layers:.1f} us per layer, {ms_eager*1e3:.0f} us launched eagerly); "
        f"{(kv_bytes + w_bytes)/1e9:.2f} GB of KV + weights -> {r['GBps']:.0f} GB/s; "
        f"{S / ms * 1e3:.0f} tokens/s bound from attention blocks alone")
    return [r]


def overlap_bench(torch):
    """How far matrix and vector instructions overlap on a gfx950 SIMD: the register-only
    probe kernels of eidola_amd/csrc/probe_overlap.hip (one iteration = the 18 MFMAs and the
    softmax vector work of one 16-row tile stage of the prefill kernel), one workgroup per CU.
    Per mode and waves per SIMD: ns per iteration (HIP events), core cycles per iteration and
    the core clock the waves saw (s_memtime against the 100 MHz s_memrealtime)."""
    import ctypes as C
    path = os.path.join(ROOT, "eidola_amd", "csrc", "libeid_probe.so")
    lib = C.CDLL(path)
    lib.eid_probe_overlap.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                      C.c_void_p]
    lib.eid_probe_overlap.restype = C.c_int
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rounds = 8                      # workgroups per CU, resident one at a time (LDS-limited)
    wgs = cus * rounds
    out = torch.empty(wgs * 512, dtype=torch.float32, device="cuda:0")
    clk = torch.zeros(wgs * 8 * 2, dtype=torch.int64, device="cuda:0")
    iters = 4000
    names = {0: "mfma_only", 1: "valu_only", 2: "phases", 3: "interleaved", 4: "role_split",
             5: "mfma_only_32x32x16", 6: "interleaved_32x32x16", 7: "tile_stage_32x32x16",
             8: "tile_stage_branches", 9: "tile_stage_branches_lds", 10: "tile_stage_no_score_chain",
             11: "tile_stage_scores_not_to_valu", 12: "tile_stage_p_not_to_mfma",
             13: "tile_stage_scores_early", 14: "tile_stage_chain_3_apart", 15: "tile_stage_chain_first"}
    res = []
    st = torch.cuda.current_stream().cuda_stream
    for mode in (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15):
        for wps in ((2,) if mode == 4 else (1, 2)):
            def run(i):
                rc = lib.eid_probe_overlap(mode, wps, wgs, iters, out.data_ptr(), clk.data_ptr(), st)
                assert rc == 0, rc
            run(0)
            ms = event_ms(run, 3, torch)
            waves = wgs * (8 if (mode == 4 or wps == 2) else 4)
            c = clk[:2 * waves].view(-1, 2).double()
            cyc = c[:, 0].mean().item() / iters
            mhz = (c[:, 0] / c[:, 1]).mean().item() * 100.0
            r = {"config": f"overlap_probe_{names[mode]}_{wps}wps", "mode": names[mode],
                 "waves_per_simd": wps, "ns_per_iter": ms * 1e6 / (iters * rounds), "cycles_per_iter": cyc,
                 "core_mhz": mhz}
            if mode == 4:
                cm = clk[:2 * waves].view(wgs, 8, 2).double()
                r["cycles_per_iter_mfma_waves"] = cm[:, :4, 0].mean().item() / iters
                r["cycles_per_iter_valu_waves"] = cm[:, 4:, 0].mean().item() / iters
            log(f"[bench] overlap probe {names[mode]:>22s}, {wps} wave(s)/SIMD: {r['ns_per_iter']:7.1f} ns "
                f"= {cyc:7.1f} cycles per iteration at {mhz:6.0f} MHz"
                + (f" (MFMA waves {r['cycles_per_iter_mfma_waves']:.1f}, vector waves "
                   f"{r['cycles_per_iter_valu_waves']:.1f} cycles)" if mode == 4 else ""))
            res.append(r)
    return res


def gather_bench(torch, ea, synth, np):
    """What a pure gather of config 2's pages sustains (eidola_amd/csrc/probe_gather.hip): the
    decode kernel's access pattern and grid shapes with no attention arithmetic, against the
    same 300,000-page pools and the same rotated page sets, so the decode kernel's 491.7 MB per
    launch can be read against what the memory system gives a kernel that only loads."""
    import ctypes as C
    lib = C.CDLL(os.path.join(ROOT, "eidola_amd", "csrc", "libeid_probe.so"))
    lib.eid_probe_gather.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                     C.c_void_p, C.c_void_p]
    lib.eid_probe_gather.restype = C.c_int
    w = Workload(lambda off: synth.config2(perm_offset=off), 8, 7, torch, ea, synth, "decode")
    sink = torch.zeros(4, dtype=torch.int32, device="cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    res = []
    tables, npages = {}, None
    for kind in ("shuffled", "contiguous"):
        per_set = []
        for s, b in enumerate(w.batches):
            nblk = (b.seq_lens.astype(np.int64) + 15) // 16
            pages = np.concatenate([b.block_table[q, :n] for q, n in enumerate(nblk)]).astype(np.int32)
            if kind == "contiguous":
                pages = np.arange(s * len(pages), (s + 1) * len(pages), dtype=np.int32)
            per_set.append(torch.from_numpy(pages).to("cuda:0"))
        tables[kind], npages = per_set, len(per_set[0])
        tables[kind + "_x8"] = [torch.cat([t[:npages // 32 * 32] for t in per_set])]
    for kind, ppw, delay, lds, rows in (
            ("shuffled", 32, 0, 75, 0), ("shuffled", 32, 0, 0, 0), ("shuffled", 16, 0, 75, 0), ("shuffled", 64, 0, 75, 0),
            ("contiguous", 32, 0, 75, 0), ("shuffled", 32, 40, 75, 0), ("shuffled", 32, 128, 75, 0),
            ("shuffled", 32, 0, 75, 1), ("shuffled", 32, 0, 0, 1), ("contiguous", 32, 0, 75, 1), ("contiguous", 32, 0, 0, 1),
            ("shuffled_x8", 32, 0, 75, 0), ("shuffled_x8", 32, 0, 75, 1), ("contiguous_x8", 32, 0, 75, 1),
            # the same with the non-temporal hint on the loads (2: whole rows, 3: head slices), and
            # one workgroup per CU as the decode kernel's even split launches them
            ("shuffled", 32, 0, 75, 2), ("shuffled", 32, 0, 75, 3), ("shuffled", 58, 0, 150, 2), ("shuffled", 58, 0, 150, 0),
            ("shuffled_x8", 32, 0, 75, 2), ("shuffled_x8", 32, 0, 75, 3), ("shuffled_x8", 58, 0, 150, 2)):
        nwg = npages // ppw
        if kind.endswith("_x8"):  # all eight page sets in one launch: the rate without the ends
            nwg *= w.n

        def run(i):
            rc = lib.eid_probe_gather(w.k_cache.data_ptr(), w.v_cache.data_ptr(),
                                      tables[kind][i % len(tables[kind])].data_ptr(), nwg, ppw, delay, lds * 1024, rows, sink.data_ptr(), st)
            assert rc == 0
        for i in range(10):
            run(i)
        ms = event_ms(run, 100, torch)
        nbytes = nwg * ppw * 2 * 16384
        shape = ("one head", "whole rows", "whole rows, non-temporal", "one head, non-temporal")[rows]
        r = {"config": f"gather_probe_{kind}_{ppw}_pages_per_wg_delay_{delay}_lds_{lds}k_{shape.replace(', ', '_').replace(' ', '_')}", "ms": ms, "bytes": nbytes,
             "GBps": nbytes / ms / 1e6, "workgroups": nwg}
        log(f"[bench] gather probe, {kind} pages, {ppw} per workgroup ({nwg} workgroups, {lds} KiB LDS, a wave reads {shape}), {delay} ALU "
            f"links per batch: {ms*1e3:.1f} us for {nbytes/1e6:.1f} MB = {r['GBps']:.0f} GB/s = {100*r['GBps']/HBM_PEAK_GBS:.1f}% of peak")
        res.append(r)
    # the same access patterns against pages that stay in cache (64 distinct pages, 2 MiB of K and
    # V): what one CU's vector memory path takes in per unit of time, by the shape of a wave's read
    rng = np.random.default_rng(1)
    for nwg, rows in ((256, 0), (256, 1), (1, 0), (1, 1)):
        ppw = 256
        tab = torch.from_numpy(rng.integers(0, 64, size=nwg * ppw, dtype=np.int32)).to("cuda:0")

        def run_c(i):
            assert lib.eid_probe_gather(w.k_cache.data_ptr(), w.v_cache.data_ptr(), tab.data_ptr(), nwg, ppw, 0,
                                        75 * 1024, rows, sink.data_ptr(), st) == 0
        for i in range(3):
            run_c(i)
        ms = event_ms(run_c, 10, torch)
        nbytes = nwg * ppw * 2 * 16384
        per_cu = nbytes / ms / 1e6 / min(nwg, 256)
        log(f"[bench] gather probe, 64 cache-resident pages, {nwg} workgroups, a wave reads "
            f"{'whole rows' if rows else 'one head'}: {ms*1e3:.1f} us = {per_cu:.1f} GB/s per CU")
        res.append({"config": f"gather_probe_cached_{nwg}_wg_{'rows' if rows else 'heads'}", "ms": ms,
                    "GBps_per_cu": per_cu})
    # LDS fragment reads (probe_lds.hip)
    lib.eid_probe_lds_read.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.eid_probe_lds_read.restype = C.c_int
    iters = 2000
    for mode, name in ((0, "linear"), (1, "128-byte rows, permuted segments"), (2, "144-byte rows")):
        for threads in (256, 512, 1024):
            def run_l(i):
                assert lib.eid_probe_lds_read(mode, 256, threads, iters, sink.data_ptr(), st) == 0
            run_l(0)
            ms = event_ms(run_l, 3, torch)
            per_cu = iters * 16 * (threads // 64) * 1024 / ms / 1e6  # GB/s
            log(f"[bench] LDS read probe, {name}, {threads // 64} waves per CU: {ms*1e3:.1f} us, "
                f"{per_cu:.0f} GB/s per CU = {per_cu / 2.4:.0f} B/clk at 2.4 GHz")
            res.append({"config": f"lds_read_probe_mode{mode}_{threads}", "ms": ms, "GBps_per_cu": per_cu})
    return res


def shim_bench(torch):
    """The engine shim's synthetic stack (8 attention blocks) under concurrent requests: the same
    16 generations (prompts of 100...1,600 bytes, 48 new tokens each) one at a time and all at
    once, i.e. what sharing steps between requests buys."""
    import threading
    from eidola_amd import engine_shim as shim
    eng = shim.SyntheticAttentionEngine(layers=8, ctx=4096, seed=1, max_seqs=16)
    prompts = [shim.render_prompt([{"role": "user", "content": "x" * (100 * (i + 1))}]) for i in range(16)]
    list(eng.generate(prompts[0], 4))       # warm-up
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_seq = sum(len(list(eng.generate(p, 48))) for p in prompts)
    t_seq = time.perf_counter() - t0
    counts = [0] * len(prompts)

    def run(i):
        counts[i] = len(list(eng.generate(prompts[i], 48)))
    steps0 = eng.steps
    t0 = time.perf_counter()
    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(prompts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    t_par = time.perf_counter() - t0
    log(f"[bench] engine shim, 16 requests x 48 new tokens, 8 attention blocks: one at a time {t_seq*1e3:.0f} ms "
        f"({n_seq / t_seq:.0f} tokens/s), all at once {t_par*1e3:.0f} ms ({sum(counts) / t_par:.0f} tokens/s) in "
        f"{eng.steps - steps0} shared steps, up to {eng.max_step_seqs} sequences per step")
    return [{"config": "engine_shim_16_requests", "sequential_s": t_seq, "concurrent_s": t_par,
             "tokens": sum(counts), "steps": eng.steps - steps0}]


def timeline_bench(torch, ea, synth, np):
    """Per-workgroup timeline of the prefill kernel on config 3's prefill rows (host-listed
    tiles) from the library's measurement aid (eid_debug_set_timeline): when workgroups start
    and end, how their duration depends on their work (least squares: fixed cost + cost per
    64-token chunk), the stamps inside the kernel, how busy the device's workgroup slots are
    over the kernel's span and how long the tail is."""
    from eidola_amd import _lib
    lib = _lib.load_measure_library()   # (the timeline hook exists in the measurement build only)
    res = []

    def one(name, w, waves, unit_name, slots_per_cu):
        attn = [c.bound_to(lib) for c in w.attn]
        n_rec = 1 << 17
        buf = torch.zeros(n_rec * 8, dtype=torch.int64, device="cuda:0")
        for i in range(300):   # (past the clock's settling time)
            attn[i % w.n]()
        torch.cuda.synchronize()
        lib.eid_debug_set_timeline(buf.data_ptr(), n_rec)
        try:
            runs = []
            for rep in range(3):
                buf.zero_()
                for i in range(20):   # the last of back-to-back calls is the one recorded
                    attn[(rep + i) % w.n]()
                torch.cuda.synchronize()
                runs.append(buf.view(-1, 8).cpu().numpy().copy())
        finally:
            lib.eid_debug_set_timeline(None, 0)
        r = runs[-1]
        used = (r[:, 0] != 0) & (r[:, 1] != 0)
        nwg = (np.nonzero(used)[0].max() // waves) + 1
        r = r[:nwg * waves].reshape(nwg, waves, 8)
        ok = (r[:, :, 0] != 0) & (r[:, :, 1] != 0)
        live = ok.any(axis=1)
        t0 = np.where(ok, r[:, :, 0], np.iinfo(np.int64).max).min(axis=1)[live]
        t1 = np.where(ok, r[:, :, 1], 0).max(axis=1)[live]
        work = (np.where(ok, r[:, :, 2] >> 32, 0).max(axis=1))[live].astype(np.float64)
        hw = r[:, 0, 2][live] & 0xffffffff
        marks = None
        if (r[:, :, 4:7][ok] != 0).all():   # stamps inside the kernel (prefill): mean over the waves
            rel = np.where(ok[:, :, None], r[:, :, 4:7] - r[:, :, 0:1], 0).sum(axis=1) / np.maximum(1, ok.sum(axis=1))[:, None]
            tail = np.where(ok, r[:, :, 1] - r[:, :, 6], 0).sum(axis=1) / np.maximum(1, ok.sum(axis=1))
            marks = np.concatenate([rel[live], tail[live][:, None]], axis=1) / 100.0
        xcc = r[:, 0, 3][live] & 0xf
        cu_key = xcc * 4096 + ((hw >> 8) & 0xff)        # XCC, then shader engine / array / CU bits
        base = t0.min()
        start = (t0 - base) / 100.0                       # microseconds (100 MHz ticks)
        end = (t1 - base) / 100.0
        dur = end - start
        span = end.max()
        A = np.stack([np.ones_like(work), work], axis=1)
        coef, *_ = np.linalg.lstsq(A, dur, rcond=None)
        ncu = len(np.unique(cu_key))
        slots = ncu * slots_per_cu
        pct = lambda q: float(np.percentile(end, q))
        out = {"config": f"timeline_{name}", "workgroups": int(live.sum()), "cus_seen": int(ncu),
               "span_us": float(span), "start_us_p50": float(np.percentile(start, 50)),
               "start_us_first_fill_max": float(np.sort(start)[min(slots, len(start)) - 1]),
               "start_us_max": float(start.max()),
               "dur_us_min": float(dur.min()), "dur_us_mean": float(dur.mean()), "dur_us_max": float(dur.max()),
               f"fit_us_fixed": float(coef[0]), f"fit_us_per_{unit_name}": float(coef[1]),
               "work_units_total": float(work.sum()), "work_units_max": float(work.max()),
               "slot_busy_frac": float(dur.sum() / (slots * span)),
               "end_us_p50": pct(50), "end_us_p90": pct(90), "end_us_p99": pct(99),
               "xcc_busy_us": [float(dur[xcc == x].sum() / max(1, len(np.unique(cu_key[xcc == x])) * slots_per_cu))
                               for x in range(8)]}
        if marks is not None:
            loop = marks[:, 2] - marks[:, 1]
            out.update({"to_first_fetch_us": float(marks[:, 0].mean()), "first_tile_us": float((marks[:, 1] - marks[:, 0]).mean()),
                        "loop_us_per_chunk": float((loop / np.maximum(work, 1)).mean()),
                        "epilogue_us": float(marks[:, 3].mean())})
            log(f"[bench] timeline {name}: per wave, start -> first fetch {out['to_first_fetch_us']:.2f} us, "
                f"first tile in LDS after {out['first_tile_us']:.2f} us more, loop {out['loop_us_per_chunk']:.3f} us per "
                f"chunk, last chunk -> end {out['epilogue_us']:.2f} us")
        try:
            np.savez(os.path.join(ROOT, "gpurun_out", f"timeline_{name}.npz"), start=start, end=end,
                     work=work, xcc=xcc, hw=hw, marks=marks if marks is not None else np.zeros(0),
                     records=r[live])
        except OSError:
            pass
        log(f"[bench] timeline {name}: {out['workgroups']} workgroups on {ncu} CUs, span {span:.1f} us; first fill "
            f"started by {out['start_us_first_fill_max']:.1f} us, last start {start.max():.1f}; duration "
            f"{dur.min():.1f}/{dur.mean():.1f}/{dur.max():.1f} us (min/mean/max) = {coef[0]:.2f} + {coef[1]:.3f} per "
            f"{unit_name}; slots busy {100*out['slot_busy_frac']:.1f}% of span; ends p50/p90/p99/max "
            f"{pct(50):.1f}/{pct(90):.1f}/{pct(99):.1f}/{span:.1f} us")
        res.append(out)

    full = lambda off: synth.config3(perm_offset=off)
    wp = Workload(lambda off: subset(full(off), np.arange(8), "config3_prefill_rows", synth), 2, 8,
                  torch, ea, synth, "varlen")
    one("config3_prefill_rows", wp, 4, "chunk", 2)
    return res


def cpu_baseline(w, torch, synth, threads):
    """The CPU restatement (oracle, fp32 path) timed on this host over the same batch:
    one full pass over page set 0 of the decode configuration."""
    import numpy as np
    import oracle
    import eidola_amd as ea
    b = w.batches[0]
    nblk = (b.seq_lens.astype(np.int64) + 15) // 16
    pages = np.concatenate([b.block_table[s, :n] for s, n in enumerate(nblk)])
    idx = torch.from_numpy(pages.astype(np.int64)).to("cuda:0")

    def host(t):
        t = t[idx].cpu().contiguous()
        return t.numpy() if t.dtype == torch.uint8 else t.view(torch.int16).numpy().view(np.uint16)

    kc, vc = host(w.k_cache), host(w.v_cache)
    bt = np.zeros((b.num_seqs, int(nblk.max())), np.int32)
    off = 0
    for s, n in enumerate(nblk):
        bt[s, :n] = np.arange(off, off + n)
        off += int(n)
    d = ea.make_desc(b.geom, num_seqs=b.num_seqs, num_q_tokens=b.num_q_tokens,
                     max_q_len=b.max_q_len, max_kv_len=b.max_kv_len,
                     max_blocks_per_seq=bt.shape[1], num_blocks=len(pages))
    q = w.q.cpu().view(torch.int16).numpy().view(np.uint16)
    sinks = w.sinks.cpu().numpy()
    ks = w.k_scale.cpu().numpy() if w.k_scale is not None else None
    vs = w.v_scale.cpu().numpy() if w.v_scale is not None else None
    args = (d, q, kc, vc, bt, b.seq_lens, b.cu_seqlens_q, sinks, ks, vs)
    oracle.attn_bf16(*args, num_threads=threads)           # warm-up (page-in, thread pool)
    reps, t0 = 0, time.time()
    while True:
        out, _ = oracle.attn_bf16(*args, num_threads=threads)
        reps += 1
        if time.time() - t0 > 10.0 or reps >= 1000:
            break
    dt = (time.time() - t0) / reps
    # cross-check while we are here: GPU result of set 0 against the CPU path
    gpu = w.attn[0]().cpu().view(torch.int16).numpy().view(np.uint16)
    err = np.abs(synth.bf16_bits_to_f32(gpu).astype(np.float64)
                 - synth.bf16_bits_to_f32(out).astype(np.float64))
    work = synth.algorithmic_work(b)
    model, ident = "", {}
    try:
        for ln in open("/proc/cpuinfo"):
            key = ln.split(":", 1)[0].strip()
            if key == "model name" and not model:
                model = ln.split(":", 1)[1].strip()
            if key in ("vendor_id", "cpu family", "model", "stepping") and key not in ident:
                ident[key] = ln.split(":", 1)[1].strip()
            if len(ident) == 4 and model:
                break
    except OSError:
        pass
    # (virtual machines often report a shortened model name: the family / model / stepping say which part it is)
    model = f"{model} ({ident.get('vendor_id', '?')} family {ident.get('cpu family', '?')} model " \
            f"{ident.get('model', '?')} stepping {ident.get('stepping', '?')})"
    return {"value": work["bytes"] / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "nproc": os.cpu_count(), "omp_num_threads_env": os.environ.get("OMP_NUM_THREADS"),
            "cpu_model": model,
            "sample": f"{reps} full passes of the same 64-sequence decode batch "
                      f"({work['ctx_tokens']} context tokens), {dt:.3f} s each, {reps*dt:.1f} s in all; "
                      "CPU restatement of this repo (no reference CPU path exists)",
            "tokens_per_s": work["q_tokens"] / dt,
            "gpu_vs_cpu_max_abs_diff": float(err.max())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=8, help="disjoint page sets rotated between steps")
    ap.add_argument("--all", action="store_true", help="also measure the other configurations")
    ap.add_argument("--report", default=os.path.join(ROOT, "gpurun_out", "bench_all.jsonl"))
    ap.add_argument("--no-cpu", action="store_true",
                    help="skip the cpu_baseline leg (CPU timing and the sampled checks against it)")
    ap.add_argument("--headline-only", action="store_true",
                    help="measure configs[1] (full attention) only, not the other configurations")
    ap.add_argument("--partition", type=int, default=0)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 1 GiB device copies (a kernel of known traffic, for "
                         "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--no-shuffle", action="store_true",
                    help="experiment: physically contiguous pages instead of a shuffled pool")
    ap.add_argument("--no-hint", action="store_true",
                    help="experiment: no host-side lengths for the library (desc.sum_kv_len = 0, no "
                         "seq_lens_host): the kernels size and plan the launch themselves")
    ap.add_argument("--only", default="",
                    help="with --all: comma-separated subset of 2w,3,4,5,sched,rope,oproj,prefill,small,stack,overlap,gather,timeline,shim "
                         "(default: everything), e.g. to profile one configuration")
    ap.add_argument("--unfused", action="store_true",
                    help="decode steps as two launches (eid_kv_write, then eid_attn_decode) "
                         "instead of one eid_attn_decode call that takes k_new / v_new")
    a = ap.parse_args()
    global NO_HINT, UNFUSED
    NO_HINT = a.no_hint
    UNFUSED = a.unfused
    if a.gpus != 1:
        sys.exit("bench.py: this path runs on ONE MI355X (no sharding, no collectives); "
                 "--gpus must be 1")
    import torch
    import eidola_amd as ea
    from eidola_amd import synth
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    ea.load_library()

    w = Workload(lambda off: synth.config2(perm_offset=off, shuffle=not a.no_shuffle)
                 .with_geom(partition_size=a.partition),
                 a.sets, 7, torch, ea, synth, "decode")
    r = measure(w, a.steps, a.warmup, torch, synth, "config2_decode_full")
    split_ms = r["ms_split"]
    kernel_ms = split_kernel_dispatch_ms(w, a.steps, torch, ea)
    achieved = r["alg_bytes"] / (kernel_ms or split_ms) / 1e6
    if kernel_ms:
        log(f"[bench] split-KV kernel by the events on its own dispatch: {kernel_ms*1e3:.1f} us = "
            f"{achieved:.0f} GB/s = {100*achieved/HBM_PEAK_GBS:.1f}% HBM (launch span with the gap before it: "
            f"{split_ms*1e3:.1f} us)")
    kernel_name = "splitkv_even_kernel<1,bf16,8 waves,direct-to-LDS loads>"
    line = {
        "metric": METRIC, "value": r["step_GBps"], "unit": "GB/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded ragged batch, N(0,1) bf16 Q/K/V and sinks, random-permuted pages)",
        "config": {"workload": "configs[1] decode continuous batch, full attention: 64 seqs, "
                               "ctx U[1,8192], Hq64/Hkv8/D64, block 16, 300k-block pool; "
                               "step = KV write of the 64 new tokens + split-KV decode + LSE merge"
                               + ("" if a.unfused else " (one eid_attn_decode call: the write is "
                                  "fused into the split-KV launch via k_new / v_new)"),
                   "partition_size": a.partition if a.partition else "run-time (workspace planned for >= %d)"
                   % ea.partition_size(w.attn[0].desc),
                   "sum_kv_len_hint": not a.no_hint, "seq_lens_host": not a.no_hint,
                   "page_sets_rotated": a.sets},
        "pct_hbm_peak": 100 * r["step_GBps"] / HBM_PEAK_GBS,
        "tokens_per_s": r["q_tokens_per_s"], "ctx_tokens_per_s": r["ctx_tokens_per_s"],
        "breakdown_us": {"kv_write": r["ms_kv_write"] * 1e3, "attn_call": r["ms_attn"] * 1e3,
                         "merge": r["ms_merge"] * 1e3,
                         "step_as_two_launches": r["ms_per_step_two_launches"] * 1e3},
        "roofline": {"bound": "hbm", "kernel": kernel_name,
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": (TRAFFIC_BYTES_PER_LAUNCH.get(kernel_name)
                                 if a.partition == 0 and not a.no_shuffle and not a.unfused else None),
                     "alg_bytes_per_launch": r["alg_bytes"], "launch_us": (kernel_ms or split_ms) * 1e3,
                     "launch_span_us": split_ms * 1e3,
                     "how": ("HIP events attached to the split-KV kernel's own dispatch inside full steps, run "
                             "through the measurement build of the library (the same sources with -DEID_MEASURE; "
                             "hipExtLaunchKernel start / stop events): the kernel's duration; launch_span_us = "
                             "from an event before the eid_attn_decode call to the library's split_done_event "
                             "(the kernel plus the launch gap before it)") if kernel_ms else
                            ("HIP events inside full steps: before the eid_attn_decode call -> the "
                             "library's split_done_event (kernel plus the launch gap before it)")},
    }
    extra = [r]
    if not a.headline_only:
        line["configs"] = other_configs(a, torch, ea, synth, w.pool, check=not a.no_cpu)
    if a.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.all:
        only = set(x for x in a.only.split(",") if x)
        want = lambda name: not only or name in only
        w = None
        torch.cuda.empty_cache()
        if want("2w"):
            ww = Workload(lambda off: synth.config2(window=128, perm_offset=off), a.sets, 7, torch,
                          ea, synth, "decode")
            extra.append(measure(ww, a.steps, a.warmup, torch, synth, "config2_decode_w128"))
            ww = None
            torch.cuda.empty_cache()
        if want("3"):
            w3 = Workload(lambda off: synth.config3(perm_offset=off), 4, 8, torch, ea, synth, "varlen")
            r3 = measure(w3, max(20, a.steps // 4), a.warmup, torch, synth, "config3_mixed")
            lw = synth.algorithmic_work(w3.batches[0], rows="long")
            sw = synth.algorithmic_work(w3.batches[0], rows="short")
            r3["prefill_flops"], r3["decode_rows_bytes"] = lw["flops"], sw["bytes"]
            extra.append(r3)
            w3 = None
            torch.cuda.empty_cache()
        if want("4"):
            w4 = Workload(lambda off: synth.config4(num_blocks=300_000, perm_offset=off), 3, 9,
                          torch, ea, synth, "decode")
            extra.append(measure(w4, max(20, a.steps // 2), a.warmup, torch, synth,
                                 "config4_fp8_decode"))
            w4 = None
            torch.cuda.empty_cache()
        for layer in (0, 1):
            if not want("5"):
                break
            w5 = Workload(lambda off: synth.config5(layer=layer, num_blocks=900_000, perm_offset=off),
                          3, 10 + layer, torch, ea, synth, "varlen")
            extra.append(measure(w5, max(10, a.steps // 10), max(3, a.warmup // 4), torch, synth,
                                 f"config5_verify_layer{layer}"))
            w5 = None
            torch.cuda.empty_cache()
            if layer == 0:
                # BASELINE words this configuration with 512-token partitions; the same batch
                # with the partition left to the library (desc.partition_size = 0)
                w5 = Workload(lambda off: synth.config5(layer=0, num_blocks=900_000, perm_offset=off)
                              .with_geom(partition_size=0), 3, 10, torch, ea, synth, "varlen")
                extra.append(measure(w5, max(10, a.steps // 10), max(3, a.warmup // 4), torch,
                                     synth, "config5_verify_layer0_runtime_partition"))
                w5 = None
                torch.cuda.empty_cache()
        if want("sched"):
            extra.append(sched_bench(synth, ea))
        if want("rope"):
            extra.extend(rope_bench(torch, ea, synth))
        if want("oproj"):
            extra.extend(oproj_bench(torch, ea))
        if want("prefill"):
            extra.extend(prefill_bench(torch, ea, synth))
        if want("small"):
            extra.extend(small_batch_bench(torch, ea, synth))
        if want("overlap"):
            extra.extend(overlap_bench(torch))
        if want("timeline"):
            import numpy as np
            extra.extend(timeline_bench(torch, ea, synth, np))
        if want("shim"):
            extra.extend(shim_bench(torch))
        if want("gather"):
            import numpy as np
            extra.extend(gather_bench(torch, ea, synth, np))
        if want("stack"):
            extra.extend(stack_bench(torch, ea, synth, fused_qkv=False))
            extra.extend(stack_bench(torch, ea, synth))
        w = Workload(lambda off: synth.config2(perm_offset=off), 1, 7, torch, ea, synth, "decode")
    if not a.no_cpu:
        threads = min(16, os.cpu_count() or 1)
        line["cpu_baseline"] = cpu_baseline(w, torch, synth, threads)
    else:
        line["cpu_baseline"] = None
    try:
        os.makedirs(os.path.dirname(a.report), exist_ok=True)
        with open(a.report, "w") as f:
            for e in extra:
                f.write(json.dumps(e) + "\n")
    except OSError:
        pass
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
