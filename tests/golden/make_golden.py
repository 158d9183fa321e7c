"""Writes the committed known-answer vectors of the CPU oracle (tests/golden/*.npz).

Two kinds, both small:
  closed_forms.npz  inputs and answers of cases whose answer is a FORMULA evaluated here in
                    float64 from the inputs alone (never the oracle's output): one key,
                    constant values, zero query, and a two-key case with and without a window;
  config1.npz       the oracle's fp64 output and lse on BASELINE config 1 (four decodes with
                    contexts 37 / 128 / 511 / 1000, seed 0), frozen so that an edit of
                    oracle/eid_oracle.c that moves a result is noticed, plus a checksum of
                    the pages its KV write produced for these tokens.
Run from the repository root:  python tests/golden/make_golden.py
tests/test_golden.py checks that the oracle still reproduces both files."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
HERE = os.path.dirname(os.path.abspath(__file__))

from eidola_amd import synth                                   # noqa: E402
from helpers import logical_tensors, cpu_caches, oracle_out      # noqa: E402


def f64(bits):
    return synth.bf16_bits_to_f32(bits).astype(np.float64)


def closed_forms():
    """Each case: a one-sequence decode batch (seq_len L, one query row); K, V, Q, sinks given
    as bf16 bits / fp32; `want` [64 heads, 64 dims] from the closed form in float64."""
    rng = np.random.default_rng(2024)
    bits = lambda x: synth.f32_to_bf16_bits(np.asarray(x, dtype=np.float32))
    scale = 0.125
    cases = {}
    # (1) one key: out = v0 * sigmoid(s0 - sink)
    q = bits(rng.standard_normal((1, 64, 64)))
    k = bits(rng.standard_normal((1, 8, 64)))
    v = bits(rng.standard_normal((1, 8, 64)))
    sinks = f64(bits(rng.standard_normal(64))).astype(np.float32)
    s0 = scale * np.einsum("hd,hd->h", f64(q)[0], np.repeat(f64(k)[0], 8, axis=0))
    want = np.repeat(f64(v)[0], 8, axis=0) / (1.0 + np.exp(sinks.astype(np.float64) - s0))[:, None]
    cases["one_key"] = dict(L=1, window=0, q=q, k=k, v=v, sinks=sinks, want=want)
    # (2) constant values c: out = c * (1 - p_sink), p_sink = e^sink / (e^sink + sum_j e^s_j)
    L = 37
    q = bits(rng.standard_normal((1, 64, 64)))
    k = bits(rng.standard_normal((L, 8, 64)))
    c = f64(bits(rng.standard_normal((8, 64))))
    v = bits(np.broadcast_to(c, (L, 8, 64)))
    s = scale * np.einsum("hd,jhd->hj", f64(q)[0], np.repeat(f64(k), 8, axis=1))
    den = np.exp(sinks.astype(np.float64)) + np.exp(s).sum(-1)
    want = np.repeat(c, 8, axis=0) * (1.0 - np.exp(sinks.astype(np.float64)) / den)[:, None]
    cases["constant_values"] = dict(L=L, window=0, q=q, k=k, v=v, sinks=sinks, want=want)
    # (3) zero query: out = mean(V) * n / (n + e^sink)
    L = 50
    q = np.zeros((1, 64, 64), np.uint16)
    k = bits(rng.standard_normal((L, 8, 64)))
    v = bits(rng.standard_normal((L, 8, 64)))
    want = np.repeat(f64(v).mean(0), 8, axis=0) * (L / (L + np.exp(sinks.astype(np.float64))))[:, None]
    cases["zero_query"] = dict(L=L, window=0, q=q, k=k, v=v, sinks=sinks, want=want)
    # (4) window 2 over 5 keys: only the last two keys count (softmax over two scores and the sink)
    L = 5
    q = bits(rng.standard_normal((1, 64, 64)))
    k = bits(rng.standard_normal((L, 8, 64)))
    v = bits(rng.standard_normal((L, 8, 64)))
    s = scale * np.einsum("hd,jhd->hj", f64(q)[0], np.repeat(f64(k), 8, axis=1))[:, -2:]
    w = np.exp(s)
    den = np.exp(sinks.astype(np.float64)) + w.sum(-1)
    want = np.einsum("hj,jhd->hd", w, np.repeat(f64(v), 8, axis=1)[-2:]) / den[:, None]
    cases["window_two"] = dict(L=L, window=2, q=q, k=k, v=v, sinks=sinks, want=want)
    flat = {}
    for name, c in cases.items():
        for key, val in c.items():
            flat[f"{name}.{key}"] = np.asarray(val)
    np.savez_compressed(os.path.join(HERE, "closed_forms.npz"), **flat)
    return cases


def config1():
    b = synth.config1()
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    out, lse = oracle_out(b, q, kc, vc, sinks)
    # (and a checksum of the bf16 pages the oracle's kv_write produced for these tokens)
    np.savez_compressed(os.path.join(HERE, "config1.npz"), out=out.astype(np.float64), lse=lse.astype(np.float64),
                        kc_sum=np.uint64(kc.astype(np.uint64).sum()), vc_sum=np.uint64(vc.astype(np.uint64).sum()))


if __name__ == "__main__":
    closed_forms()
    config1()
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))
