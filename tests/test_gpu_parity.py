"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

Bars: KV writes bit-exact; attention outputs within max-abs 2e-2 / mean-abs 2e-3 of the
fp64 oracle (bf16 output, fp32 accumulation).  Parity is against this repository's own
oracle: the reference holds no implementation of this path."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
import eidola_amd as ea
from eidola_amd import KV_BF16, KV_FP8_E4M3, synth
from eidola_amd.ops import workspace_layout

MAX_ABS_TOL_REL, MEAN_ABS_TOL_REL = 2e-2, 2e-3   # the attention tolerances per unit of value magnitude

from helpers import (make_batch, desc_of, logical_tensors, cpu_caches, oracle_out, fp8_scales,
                     all_slots, empty_caches, assert_close)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()       # raises if the HIP extension has not been built
    return gpu_helpers


# ---------------------------------------------------------------- K1: kv_write
def test_kv_write_bf16_bit_exact_with_skips_and_poison(G):
    b = make_batch([37, 128, 511, 1000, 5], [1, 1, 1, 1, 1], num_blocks=200)
    q, k, v, _ = logical_tensors(b)
    sm = all_slots(b)
    sm[::17] = -1
    kc, vc = empty_caches(b)
    oracle.kv_write(desc_of(b), k, v, kc, vc, sm)
    kc_d, vc_d = G.cache_dev(empty_caches(b)[0]), G.cache_dev(empty_caches(b)[1])
    ea.kv_write(b.geom, G.bf16_dev(k), G.bf16_dev(v), kc_d, vc_d, G.dev(sm))
    torch.cuda.synchronize()
    assert np.array_equal(G.cache_host(kc_d), kc)
    assert np.array_equal(G.cache_host(vc_d), vc)


def test_kv_write_empty_and_all_skipped(G):
    b = make_batch([16], [1])
    kc, vc = empty_caches(b)
    kc_d, vc_d = G.cache_dev(kc), G.cache_dev(vc)
    z = torch.empty((0, 8, 64), dtype=torch.bfloat16, device=G.DEV)
    ea.kv_write(b.geom, z, z, kc_d, vc_d, torch.empty(0, dtype=torch.int64, device=G.DEV))
    q, k, v, _ = logical_tensors(b)
    ea.kv_write(b.geom, G.bf16_dev(k), G.bf16_dev(v), kc_d, vc_d,
                torch.full((16,), -1, dtype=torch.int64, device=G.DEV))
    torch.cuda.synchronize()
    assert np.array_equal(G.cache_host(kc_d), kc) and np.array_equal(G.cache_host(vc_d), vc)


@pytest.mark.parametrize("scale", [1.0, 0.0078125, 3.7e-3, 0.013671875, 123.456])
def test_kv_write_fp8_exhaustive_over_all_bf16_inputs(G, scale):
    """Every one of the 65,536 bf16 bit patterns, as K and (bit-reversed order) as V."""
    n_tok = 65536 // (8 * 64)
    b = make_batch([n_tok], [1], kv_dtype=KV_FP8_E4M3, shuffle=True)
    k = np.arange(65536, dtype=np.uint32).astype(np.uint16).reshape(n_tok, 8, 64)
    v = k[::-1].copy()
    ks = np.full(8, scale, np.float32) * np.array([1, 2, 0.5, 1, 3, 1, 7, 1], np.float32)
    vs = ks[::-1].copy()
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    torch.cuda.synchronize()
    assert np.array_equal(G.cache_host(kc_d), kc)
    assert np.array_equal(G.cache_host(vc_d), vc)


# ---------------------------------------------------------------- config 1 (plumbing)
def test_config1_plumbing_decode(G):
    b = synth.config1()
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    assert np.array_equal(G.cache_host(kc_d), kc) and np.array_equal(G.cache_host(vc_d), vc)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
    assert_close(out, ref, "config1")
    assert np.allclose(lse, ref_lse, atol=2e-3)


# ---------------------------------------------------------------- decode, ragged edge cases
@pytest.mark.parametrize("window", [0, 1, 16, 128])
@pytest.mark.parametrize("partition", [0, 64, 128, 512])
def test_decode_ragged_edges(G, window, partition):
    seq_lens = [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 500, 1024, 1500]
    b = make_batch(seq_lens, [1] * len(seq_lens), window=window, partition=partition)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
    assert_close(out, ref, f"decode w={window} P={partition}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


def test_decode_without_sinks_and_with_extreme_sinks(G):
    b = make_batch([300, 40, 700], [1, 1, 1], partition=128)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    for sk in (None, np.full(64, 30.0, np.float32), np.full(64, -30.0, np.float32)):
        ref, _ = oracle_out(b, q, kc, vc, sk)
        out = G.run_attn(b, q, kc_d, vc_d, sk)
        assert_close(out, ref, f"sinks={None if sk is None else sk[0]}")


@pytest.mark.parametrize("hkv", [8, 16])
@pytest.mark.parametrize("window,partition,host_lens", [(0, 0, False), (0, 0, True), (0, 128, True),
                                                        (200, 0, False)])
def test_fp8_decode_two_kv_heads_per_wave(G, hkv, window, partition, host_lens):
    """One query row per sequence over an fp8 cache with KV heads in groups of eight: a wave of
    the split-KV kernel serves two neighbouring KV heads (per-head scales, sinks and outputs
    must land on the right 16 query heads).  Long and short sequences, ends at every offset of
    a 32-token step, with lse; also through the host's item list."""
    seq_lens = [2100 + i for i in range(33)] + [5000, 64, 1, 31, 32, 33, 700, 9000]
    b = make_batch(seq_lens, [1] * len(seq_lens), window=window, partition=partition,
                   kv_dtype=KV_FP8_E4M3, num_kv_heads=hkv, seed=77)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v)
    ks = (ks * np.linspace(0.5, 2.0, hkv)).astype(np.float32)   # clearly different per head
    vs = (vs * np.linspace(2.0, 0.5, hkv)).astype(np.float32)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, host_lens=host_lens,
                          hint=host_lens, decode=True)
    assert_close(out, ref, f"fp8 head pairs Hkv={hkv} w={window} P={partition}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


def test_decode_two_kv_heads(G):
    b = make_batch([200, 33], [1, 1], num_kv_heads=2, partition=64)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, "Hkv=2")


def test_decode_is_invariant_under_page_permutation_bitwise(G):
    seq_lens = [700, 45, 1030]
    a = make_batch(seq_lens, [1, 1, 1], seed=21, partition=256)
    c = make_batch(seq_lens, [1, 1, 1], seed=22, num_blocks=400, partition=256)
    q, k, v, sinks = logical_tensors(a, seed=5)
    outs = []
    for b in (a, c):
        kc_d, vc_d = G.gpu_caches(b, k, v)
        outs.append(G.run_attn(b, q, kc_d, vc_d, sinks))
    assert np.array_equal(outs[0], outs[1])


def test_garbage_beyond_sequence_end_is_never_used(G):
    """Slots past seq_len inside the last page hold NaN patterns (poison) in K and V."""
    b = make_batch([33, 100], [1, 1])
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)              # unwritten slots stay 0x7FC1 (NaN)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, "poison tail")


def test_prefill_rows_never_use_garbage_beyond_sequence_end(G):
    """The prefill kernel loads whole 64-token tiles: the rows of a tile past seq_len (unwritten
    slots of the last page, NaN patterns here, and pages the table does not even hold) must not
    reach the output, with and without an lse (the two softmax variants load tiles differently)."""
    b = make_batch([45, 100, 333, 1000], [40, 64, 200, 9])
    q, k, v, sinks = logical_tensors(b, seed=31)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, lse = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, "prefill poison tail")
    out, lse_gpu = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
    assert_close(out, ref, "prefill poison tail, lse asked for")
    assert np.all(np.isfinite(lse_gpu))


# ---------------------------------------------------------------- varlen: verify rows
@pytest.mark.parametrize("window", [0, 128])
@pytest.mark.parametrize("partition", [0, 512])
def test_verify_five_rows(G, window, partition):
    seq_lens = [5, 21, 130, 517, 1029, 2300]
    b = make_batch(seq_lens, [5] * len(seq_lens), window=window, partition=partition)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
    assert_close(out, ref, f"verify w={window} P={partition}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("window,partition,seq_lens,q_lens,host_lens", [
    (0, 0, [3000, 700, 5000, 90, 8], [8, 7, 3, 1, 8], False),        # small batch: 512-key partitions
    (0, 256, [3000, 700, 5000, 90], [8, 7, 5, 2], False),            # the caller's partition
    (128, 0, [3000, 700, 150, 9], [8, 7, 8, 7], True),               # windowed: short spans
    (0, 0, [1200 + 37 * i for i in range(40)], [7, 8] * 20, True),   # split-KV kernel, host plan
    (0, 0, [900 + 53 * i for i in range(70)], [8] * 70, False),      # one class only, run-time rule
    (0, 0, [3000, 700, 5000, 90, 16], [16, 9, 3, 1, 16], False),     # 9..16 rows: two waves per KV head
    (0, 256, [3000, 700, 5000, 90], [12, 16, 5, 2], True),
    (128, 0, [3000, 700, 150, 13], [16, 10, 8, 13], True),           # ... windowed (one partition each)
    (0, 0, [1200 + 37 * i for i in range(40)], [16, 11] * 20, True),
    (0, 0, [900 + 53 * i for i in range(70)], [16] * 70, False),     # too many for that: prefill kernel
    (0, 0, [3000, 700, 5000, 90, 32], [32, 17, 3, 1, 32], False),    # 17..32 rows: four waves per KV head
    (0, 256, [6000, 2100], [20, 25], True),
    (128, 0, [3000, 700, 150, 30, 400, 77, 900, 64], [32, 20, 8, 30, 1, 17, 24, 2], True),
])
def test_seven_and_eight_query_rows_take_four_tiles(G, kv_dtype, window, partition, seq_lens,
                                                    q_lens, host_lens):
    """When no sequence of the batch has more than 8 query rows, sequences of 7 and 8 rows
    stay in the split-KV class (64 rows = four 16-row tiles per KV head) instead of going to
    the prefill kernel; up to 16 rows, two waves share a KV head (8 query tokens each).
    Against the oracle, with lse, for every kernel that serves the class."""
    b = make_batch(seq_lens, q_lens, window=window, partition=partition, kv_dtype=kv_dtype)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, host_lens=host_lens,
                          hint=host_lens)
    assert_close(out, ref, f"q_len 7..8 w={window} P={partition}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


@pytest.mark.parametrize("q_lens,partition,host_lens,window", [
    ([3, 4, 5, 6] * 10, 128, True, 0),    # three row tiles, the host's ranges
    ([5] * 40, 0, False, 0),              # ... ranges found on the device
    ([6, 3] * 20, 128, False, 0),
    ([7, 8] * 20, 128, True, 0),          # four row tiles
    ([8] * 40, 0, False, 0),
    ([4, 5] * 30, 128, True, 3000),       # a window that starts inside a page and a chunk
])
def test_verify_rows_over_an_fp8_cache_on_the_even_split(G, q_lens, partition, host_lens, window):
    """A verify batch over an fp8 cache that is large enough for the even split (equal ranges of
    chunks per workgroup): one KV head per wave, the chunks' raw bytes streamed into LDS and the
    V operands read transposed from the bytes.  Ragged lengths (tails inside a page and inside
    a chunk), against the oracle with lse."""
    rng = np.random.default_rng(len(q_lens) + partition + sum(q_lens))
    seq_lens = rng.integers(1500, 9000, size=len(q_lens))
    b = make_batch(seq_lens, q_lens, window=window, partition=partition, kv_dtype=KV_FP8_E4M3)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, host_lens=host_lens,
                          hint=host_lens)
    assert_close(out, ref, f"fp8 verify rows, even split, P={partition} w={window}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


def test_eighth_row_agrees_with_the_prefill_kernel(G):
    """The same 8-row sequences once in a batch whose longest query is 8 rows (split-KV class,
    four tiles) and once next to a 9-row sequence (then they are prefill rows): two kernels,
    one result within rounding."""
    L, ql = [2500, 900, 4000], [8, 7, 8]
    b8 = make_batch(L, ql, seed=3)
    b9 = make_batch(L + [600], ql + [9], seed=3)
    q, k, v, sinks = logical_tensors(b9)
    kc_d, vc_d = G.gpu_caches(b9, k, v)
    o9 = G.run_attn(b9, q, kc_d, vc_d, sinks)
    b8.block_table[:, :] = b9.block_table[:3, :b8.block_table.shape[1]]
    o8 = G.run_attn(b8, q[:23], kc_d, vc_d, sinks)
    a = synth.bf16_bits_to_f32(o8).astype(np.float64)
    c = synth.bf16_bits_to_f32(o9[:23]).astype(np.float64)
    assert np.abs(a - c).max() <= 4e-3


def test_sixteen_rows_agree_with_the_prefill_kernel(G):
    """9..16-row sequences through the row-split split-KV kernel, and the same sequences
    next to a 17-row one (prefill kernel): one result within rounding."""
    L, ql = [2500, 900, 4000, 300], [16, 9, 12, 16]
    bs = make_batch(L, ql, seed=5)
    bl = make_batch(L + [600], ql + [17], seed=5)
    q, k, v, sinks = logical_tensors(bl)
    kc_d, vc_d = G.gpu_caches(bl, k, v)
    ol = G.run_attn(bl, q, kc_d, vc_d, sinks)
    bs.block_table[:, :] = bl.block_table[:4, :bs.block_table.shape[1]]
    n = sum(ql)
    os_ = G.run_attn(bs, q[:n], kc_d, vc_d, sinks)
    a = synth.bf16_bits_to_f32(os_).astype(np.float64)
    c = synth.bf16_bits_to_f32(ol[:n]).astype(np.float64)
    assert np.abs(a - c).max() <= 4e-3


def test_verify_row_equals_decode_row(G):
    L = 777
    b5 = make_batch([L], [5], partition=256)
    q, k, v, sinks = logical_tensors(b5)
    kc_d, vc_d = G.gpu_caches(b5, k, v)
    out5 = synth.bf16_bits_to_f32(G.run_attn(b5, q, kc_d, vc_d, sinks))
    for t in (0, 4):
        b1 = make_batch([L - 4 + t], [1], partition=256)
        k1, v1 = k[:L - 4 + t], v[:L - 4 + t]
        kc1, vc1 = G.gpu_caches(b1, k1, v1)
        out1 = synth.bf16_bits_to_f32(G.run_attn(b1, q[t:t + 1], kc1, vc1, sinks))
        assert np.abs(out5[t] - out1[0]).max() <= 1e-2


@pytest.mark.parametrize("window", [0, 40])
def test_varlen_mixed_short_lengths(G, window):
    seq_lens = [9, 64, 300, 31, 1000, 6, 450]
    q_lens = [1, 2, 3, 4, 5, 6, 1]
    b = make_batch(seq_lens, q_lens, window=window, partition=128)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, f"mixed short w={window}")


# ---------------------------------------------------------------- varlen: prefill chunks
@pytest.mark.parametrize("window", [0, 128])
def test_prefill_chunks_and_decodes_mixed(G, window):
    seq_lens = [7, 40, 100 + 64, 512, 300 + 512, 1, 200, 33]
    q_lens = [7, 40, 64, 512, 512, 1, 1, 5]
    b = make_batch(seq_lens, q_lens, window=window)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
    assert_close(out, ref, f"prefill mixed w={window}")
    assert np.allclose(lse, ref_lse, atol=2e-3)
    # without lse the prefill kernel folds the softmax factor into its Q operands
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, f"prefill mixed w={window}, no lse")


@pytest.mark.parametrize("shape", ["rising", "falling", "deep", "spikes"])
@pytest.mark.parametrize("window", [0, 100])
def test_prefill_scores_far_from_zero(G, shape, window):
    """Scores that climb by tens of log2 units per 64-key chunk (the reference of the prefill
    kernel's softmax is outgrown again and again: its row-sum guard has to trip and recover),
    fall as fast (later chunks underflow against it), sit some 70 log2 units below zero
    throughout (a row's first maximum is far from the value its accumulator starts at), or
    are ordinary except for single keys of some KV heads that score ~130 log2 units higher
    (only some rows of some chunks overflow).  Prefill rows and a few decode / verify rows,
    with lse (unfolded softmax factor) and without (factor folded into the Q operands)."""
    seq_lens, q_lens = [600, 333, 64, 700, 90], [64, 333, 64, 5, 1]
    b = make_batch(seq_lens, q_lens, window=window, seed=61)
    q, k, v, sinks = logical_tensors(b)
    qf = synth.bf16_bits_to_f32(q) * np.float32(0.5)
    kf = synth.bf16_bits_to_f32(k) * np.float32(0.5)
    # a common offset on all 64 dims: q.k grows by 64 * (q offset) * (k offset), times 1/8
    pos = np.concatenate([np.arange(L, dtype=np.float32) for L in seq_lens])[:, None, None]
    if shape == "rising":        # + 0.5 nats per key position: 32 nats = 46 log2 units per chunk
        qf += 1
        kf += pos / 16
    elif shape == "falling":
        qf += 1
        kf -= pos / 16
    elif shape == "deep":        # about -50 nats everywhere
        qf -= 1
        kf += np.float32(6.25)
    else:                        # q offset 1, a few keys offset 12 on two KV heads: +96 nats there
        qf += 1
        rng = np.random.default_rng(5)
        hot = rng.choice(kf.shape[0], size=24, replace=False)
        kf[hot[:12], 2] += np.float32(12)
        kf[hot[12:], 5] += np.float32(12)
    q, k = synth.f32_to_bf16_bits(qf), synth.f32_to_bf16_bits(kf)
    sinks = None if shape == "deep" else sinks
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
    assert_close(out, ref, f"{shape} w={window}")
    assert np.allclose(lse, ref_lse, atol=2e-3, rtol=1e-5)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, f"{shape} w={window}, no lse")


def test_varlen_at_qlen1_equals_decode_entry_point(G):
    b = make_batch([100, 1000, 17], [1, 1, 1], partition=128)
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    a = G.run_attn(b, q, kc_d, vc_d, sinks, decode=True)
    c = G.run_attn(b, q, kc_d, vc_d, sinks, decode=False)
    assert np.array_equal(a, c)


def test_many_sequences_cross_the_64_wide_scan(G):
    """More than 64 sequences of mixed classes: the device-side work lists are built by
    64-wide prefix scans that must chain across batches."""
    rng = np.random.default_rng(3)
    S = 150
    q_lens = rng.choice([1, 1, 1, 2, 4, 5, 6, 9, 33, 70], size=S)
    seq_lens = q_lens + rng.integers(0, 700, size=S)
    for window in (0, 48):
        b = make_batch(seq_lens, q_lens, window=window)
        q, k, v, sinks = logical_tensors(b)
        kc, vc = cpu_caches(b, k, v)
        kc_d, vc_d = G.gpu_caches(b, k, v)
        ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
        out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)
        assert_close(out, ref, f"150 sequences w={window}")
        assert np.allclose(lse, ref_lse, atol=2e-3)
        assert np.array_equal(G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True, hint=True)[0], out)
        assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, hint=True), ref, f"150 sequences w={window}, no lse")


@pytest.mark.parametrize("kind", ["decode", "mixed", "uniform", "one_long"])
def test_at_least_one_sequence_per_cu(G, kind):
    """300 and more sequences.  With no span beyond 2,048 tokens the host plans every sequence
    as one work item (no partials); one longer sequence sends the batch back to the run-time
    rule (several fills, or equal pieces when the lengths are uniform)."""
    rng = np.random.default_rng(17)
    S = 300
    if kind == "decode":
        q_lens = np.ones(S, np.int64)
        seq_lens = rng.integers(1, 1300, size=S)
    elif kind == "mixed":
        q_lens = rng.choice([1, 1, 1, 2, 5, 6, 20], size=S)
        seq_lens = q_lens + rng.integers(0, 900, size=S)
    elif kind == "uniform":
        q_lens = np.ones(S, np.int64)
        seq_lens = np.full(S, 2304)            # beyond the cap: two equal pieces each
    else:
        q_lens = np.ones(S, np.int64)
        seq_lens = rng.integers(1, 700, size=S)
        seq_lens[123] = 5000
    b = make_batch(seq_lens, q_lens, seed=19)
    d = desc_of(b)
    if kind in ("decode", "mixed"):
        assert ea.partition_size(d) == (int(seq_lens.max()) + 63) // 64 * 64
    else:
        assert ea.partition_size(d) == 256      # run-time choice, planned from its lower bound
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True, hint=True)
    assert_close(out, ref, f"300 sequences, {kind}")
    assert np.allclose(lse, ref_lse, atol=2e-3)
    assert np.array_equal(G.run_attn(b, q, kc_d, vc_d, sinks, return_lse=True)[0], out)  # without the hint
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, f"300 sequences, {kind}, no lse")


def test_loose_max_kv_len_leaves_the_choice_to_the_kernels(G):
    """300 short sequences declared with max_kv_len = 4,096: the host cannot plan whole
    sequences, the kernels find out by themselves that every sequence is one item."""
    rng = np.random.default_rng(23)
    seq_lens = rng.integers(1, 700, size=300)
    b = make_batch(seq_lens, np.ones(300, np.int64), seed=29)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    bt = np.zeros((300, 256), np.int32)
    bt[:, :b.block_table.shape[1]] = b.block_table
    for hint in (0, int(seq_lens.sum())):
        out = ea.attn_decode(b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(bt), G.dev(b.seq_lens),
                             max_kv_len=4096, sinks=G.dev(sinks), sum_kv_len=hint)
        torch.cuda.synchronize()
        assert_close(G.bits_host(out), ref, f"loose bound, hint {hint}")


@pytest.mark.parametrize("hkv", [1, 4, 16])
def test_other_kv_head_counts(G, hkv):
    b = make_batch([300, 40, 1, 77], [1, 5, 1, 40], num_kv_heads=hkv, partition=128)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, f"Hkv={hkv}")


def test_prefill_from_empty_context_and_exact_page_multiples(G):
    """Chunks whose context is exactly the chunk (no prior), page- and tile-aligned or not."""
    seq_lens = [32, 64, 96, 100, 512, 7]
    b = make_batch(seq_lens, seq_lens)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, "no-prior prefill")


def test_partition_count_at_its_maximum(G):
    """Smallest partition on a long sequence: 4096/64 = 64 partitions for one row."""
    b = make_batch([4096, 4095, 65], [1, 1, 1], partition=64)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks), ref, "64 partitions")


@pytest.mark.parametrize("host_lens", [False, True])
def test_table_entries_beyond_a_sequence_do_not_matter(G, host_lens):
    """Entries of a block-table row past the sequence's last page are undefined: whatever
    they hold (here negative and huge ids), the output is the same bit for bit, through the
    short-span, split-KV and prefill kernels."""
    b = make_batch([700, 45, 3000, 1, 130, 2000], [1, 1, 5, 1, 2, 40])
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    clean = G.run_attn(b, q, kc_d, vc_d, sinks, host_lens=host_lens)
    junk = np.array([-1, 0x7fffffff, -(2 ** 31), 123456789], np.int32)
    for s_, L in enumerate(b.seq_lens):
        n = (int(L) + 15) // 16
        tail = b.block_table[s_, n:]
        tail[:] = junk[np.arange(len(tail)) % 4]
    dirty = G.run_attn(b, q, kc_d, vc_d, sinks, host_lens=host_lens)
    assert np.array_equal(clean, dirty)


def test_errors_surface_as_status_codes_on_the_gpu_box(G):
    b = make_batch([100], [1])
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    with pytest.raises(ea.EidError) as e:
        ea.attn_decode(b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                       max_kv_len=100, workspace=torch.empty(256, dtype=torch.uint8, device=G.DEV))
    assert e.value.name == "EID_ERR_WORKSPACE"
    with pytest.raises(ea.EidError) as e:   # block table too narrow for max_kv_len
        ea.attn_decode(b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                       max_kv_len=100000)
    assert e.value.name == "EID_ERR_INVALID_ARG"


# ---------------------------------------------------------------- fp8 KV
@pytest.mark.parametrize("q_len", [1, 5, 48])
def test_fp8_kv_attention(G, q_len):
    seq_lens = [130, 64, 900, 2100]
    b = make_batch(seq_lens, [q_len] * 4, kv_dtype=KV_FP8_E4M3, partition=256)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    assert np.array_equal(G.cache_host(kc_d), kc) and np.array_equal(G.cache_host(vc_d), vc)
    ref, _ = oracle_out(b, q, kc, vc, sinks, ks, vs)
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs), ref, f"fp8 q_len={q_len}")


# ---------------------------------------------------------------- short-span kernel
@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("window,seq_lens,q_lens", [
    (128, [1, 15, 16, 17, 129, 400, 1500, 3000], [1] * 8),            # windowed decode
    (0, [1, 63, 64, 65, 300, 511, 512, 7], [1, 1, 1, 1, 1, 1, 1, 2]), # short contexts, 8 chunks
    (40, [200, 77, 90, 1000], [5, 3, 6, 4]),                          # verify rows, windowed
    (64, [300, 50, 900, 12, 640], [1, 5, 2, 6, 1]),                   # classes mixed
])
def test_short_spans_one_chunk_per_wave(G, kv_dtype, window, seq_lens, q_lens):
    """No sequence spans more than 8 chunks and the batch is small: the attention entry
    points take the kernel that gives every wave one chunk and merges in LDS.  Outputs and
    lse against the oracle, for both cache types and every q_len class."""
    b = make_batch(seq_lens, q_lens, window=window, kv_dtype=kv_dtype)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True)
    assert_close(out, ref, f"short spans w={window}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("window,seq_lens,q_lens,hint", [
    (0, [4096], [1], False),                                   # one sequence, 8 partitions
    (0, [513, 1024, 1025, 2500], [1, 1, 1, 1], False),         # partition edges
    (0, [20000, 300, 64, 1], [1, 1, 2, 1], True),              # ragged, sized by the sum
    (0, [3000, 700, 5000], [5, 3, 6], False),                  # verify rows
    (2000, [6000, 2100, 900], [1, 4, 1], False),               # window wider than a partition
    (0, [2000, 1500, 116], [1, 5, 40], False),                 # next to a prefill chunk
])
def test_small_batches_in_partitions_of_512(G, kv_dtype, window, seq_lens, q_lens, hint):
    """A batch small enough that every 64-key chunk gets a wave of its own at once: the entry
    points cut the sequences into 512-key partitions, one workgroup of eight waves per
    partition and KV head, and merge the partitions afterwards.  Outputs and lse against the
    oracle; the planning is visible through eid_partition_size."""
    b = make_batch(seq_lens, q_lens, window=window, kv_dtype=kv_dtype)
    desc = desc_of(b)
    desc.sum_kv_len = int(b.seq_lens.sum()) if hint else 0
    assert ea.partition_size(desc) == 512
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, hint=hint)
    assert_close(out, ref, f"small batch w={window}")
    assert np.allclose(lse, ref_lse, atol=2e-3)


def test_small_batch_partitions_agree_with_the_split_kv_kernel(G):
    """The same four sequences through the 512-key partitions of the small-batch path
    (run-time partition) and through the split-KV kernel (the caller's partition of 256):
    two different kernels and merge inputs, one result within rounding."""
    b = make_batch([9000, 4000, 777, 512], [1] * 4, seed=12)
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    a = G.run_attn(b, q, kc_d, vc_d, sinks)
    from dataclasses import replace
    c = G.run_attn(b, q, kc_d, vc_d, sinks, geom=replace(b.geom, partition_size=256))
    fa = synth.bf16_bits_to_f32(a).astype(np.float64)
    fc = synth.bf16_bits_to_f32(c).astype(np.float64)
    assert np.abs(fa - fc).max() <= 4e-3
    kc, vc = cpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    assert_close(a, ref, "small batch, 512-key partitions")
    assert_close(c, ref, "small batch, split-KV kernel")


def test_short_span_and_split_kv_kernels_agree_across_the_fill_boundary(G):
    """64 windowed decodes fill the device exactly at one workgroup per (sequence, KV head);
    65 fall back to the split-KV kernel.  The first 64 rows must agree between the two."""
    rng = np.random.default_rng(8)
    L = rng.integers(1, 2000, size=65)
    b65 = make_batch(L, [1] * 65, window=128, seed=4)
    q, k, v, sinks = logical_tensors(b65)
    kc_d, vc_d = G.gpu_caches(b65, k, v)
    o65 = G.run_attn(b65, q, kc_d, vc_d, sinks)
    b64 = make_batch(L[:64], [1] * 64, window=128, seed=4)
    b64.block_table[:] = b65.block_table[:64]
    o64 = G.run_attn(b64, q[:64], kc_d, vc_d, sinks)
    a = synth.bf16_bits_to_f32(o64).astype(np.float64)
    c = synth.bf16_bits_to_f32(o65[:64]).astype(np.float64)
    assert np.abs(a - c).max() <= 4e-3
    kc, vc = cpu_caches(b65, k, v)
    ref, _ = oracle_out(b65, q, kc, vc, sinks)
    assert_close(o65, ref, "65 windowed decodes")
    assert_close(o64, ref[:64], "64 windowed decodes")


def test_fp8_every_code_dequantises_exactly(G):
    """One-key attention returns v0 * sigmoid(s0 - sink): with a huge negative sink the
    output is the dequantised V row itself, for all 254 finite codes."""
    n_tok = 4
    b = make_batch([1] * n_tok, [1] * n_tok, kv_dtype=KV_FP8_E4M3)
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    vc = np.zeros((b.num_blocks, 16, 8, 64), np.uint8)
    kc = np.zeros_like(vc)
    flat = vc.reshape(-1, 8 * 64)
    for s in range(n_tok):
        slot = int(b.all_slots(s)[0])
        flat[slot] = np.resize(np.roll(codes, 64 * s), 512)
    vs = np.ones(8, np.float32)
    q = np.zeros((n_tok, 64, 64), np.uint16)
    sinks = np.full(64, -100.0, np.float32)
    out = G.run_attn(b, q, G.cache_dev(kc), G.cache_dev(vc), sinks, vs, vs)
    got = synth.bf16_bits_to_f32(out).reshape(n_tok, 8, 8, 64)
    for s in range(n_tok):
        want = oracle.fp8_decode(flat[int(b.all_slots(s)[0])]).reshape(8, 1, 64)
        assert np.array_equal(got[s], np.broadcast_to(want, (8, 8, 64)))


# ---------------------------------------------------------------- K4 alone
def test_lse_merge_entry_point_against_oracle_merge(G):
    seq_lens, q_lens = [700, 1300, 90], [5, 5, 5]
    b = make_batch(seq_lens, q_lens, partition=128)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    d = desc_of(b)
    P, nparts, ws_rows, ml_off, acc_off = workspace_layout(d)
    assert P == 128 and ws_rows == 5
    ml, acc = oracle.splitkv_f64(d, P, nparts, q, kc, vc, b.block_table, b.seq_lens, b.cu_seqlens_q)
    ref, ref_lse = oracle.lse_merge_f64(ml, acc, sinks)
    full, _ = oracle_out(b, q, kc, vc, sinks)
    assert np.allclose(ref, full, rtol=1e-10, atol=1e-13)
    # workspace rows are (sequence, row-in-sequence); here every sequence has ws_rows rows
    ws = np.zeros(ea.workspace_bytes(d), np.uint8)
    # the oracle returns [row, head, partition, ...]; the workspace is [row, partition, head, ...]
    ml_ws = np.ascontiguousarray(ml.astype(np.float32).transpose(0, 2, 1, 3))
    ws[ml_off:ml_off + ml.size * 4] = ml_ws.reshape(-1).view(np.uint8)
    with np.errstate(invalid="ignore", divide="ignore"):
        o_part = np.where(ml[..., 1:2] > 0, acc / ml[..., 1:2], 0.0).astype(np.float16)
    o_ws = np.ascontiguousarray(o_part.transpose(0, 2, 1, 3))
    ws[acc_off:acc_off + o_part.size * 2] = o_ws.reshape(-1).view(np.uint8)
    ws_d = torch.from_numpy(ws).to(G.DEV)
    lse_d = torch.zeros((15, 64), dtype=torch.float32, device=G.DEV)
    out = ea.ops.lse_merge(b.geom, ws_d, G.dev(b.seq_lens), G.dev(b.cu_seqlens_q),
                           num_q_tokens=15, max_q_len=5, max_kv_len=1300,
                           max_blocks_per_seq=b.block_table.shape[1], num_blocks=b.num_blocks,
                           sinks=G.dev(sinks), lse=lse_d)
    torch.cuda.synchronize()
    # sequence 2 (90 tokens) has one partition: the merge leaves its rows to the main kernel
    assert_close(G.bits_host(out)[:10], ref[:10], "merge")
    assert np.allclose(lse_d.cpu().numpy()[:10], ref_lse[:10], atol=1e-4)
    assert (G.bits_host(out)[10:] == 0).all()


def test_split_done_event_is_recorded_between_the_phases(G):
    """args.split_done_event is a profiling hook: recorded after the split-KV launch, before
    the merge; it must not change the result."""
    b = make_batch([3000, 1500, 70], [1, 1, 1], partition=256)
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    call = ea.prepare("eid_attn_decode", b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table),
                      G.dev(b.seq_lens), max_kv_len=b.max_kv_len, sinks=G.dev(sinks))
    ref = call().clone()
    torch.cuda.synchronize()
    e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    for e in (e0, e1, e2):
        e.record()   # creates the hipEvent_t handles
    torch.cuda.synchronize()
    call.out.zero_()
    e0.record()
    call.args.split_done_event = e1.cuda_event
    call()
    e2.record()
    torch.cuda.synchronize()
    call.args.split_done_event = None
    assert torch.equal(call.out, ref)
    assert 0.0 < e0.elapsed_time(e1) <= e0.elapsed_time(e2)


@pytest.mark.parametrize("seed", range(16))
def test_seeded_random_batches(G, seed):
    """Random shapes across every dispatch decision at once: number of sequences, q_len
    classes, context lengths, window, partition mode, cache type, launch hint."""
    rng = np.random.default_rng(1000 + seed)
    S = int(rng.integers(1, 41))
    q_lens = rng.choice([1, 1, 1, 2, 3, 5, 6, 7, 20, 33, 64, 100], size=S)
    ctx = rng.integers(0, int(rng.choice([60, 400, 3000])), size=S)
    seq_lens = q_lens + ctx
    window = int(rng.choice([0, 0, 16, 128, 500]))
    partition = int(rng.choice([0, 0, 64, 256, 1024]))
    kv_dtype = KV_FP8_E4M3 if rng.random() < 0.35 else KV_BF16
    b = make_batch(seq_lens, q_lens, window=window, partition=partition, kv_dtype=kv_dtype,
                   seed=seed)
    q, k, v, sinks = logical_tensors(b)
    if rng.random() < 0.2:
        sinks = None
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True,
                          hint=bool(rng.random() < 0.5), host_lens=bool(rng.random() < 0.5))
    what = f"seed {seed}: S={S} w={window} P={partition} dtype={kv_dtype} q={sorted(set(q_lens.tolist()))}"
    assert_close(out, ref, what)
    assert np.allclose(lse, ref_lse, atol=3e-3), what
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs), ref, what + ", no lse")


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("window,partition,seq_lens,q_lens", [
    (0, 0, [5000, 300, 9000, 40, 1, 2500], [1] * 6),                 # ragged decode
    (0, 0, [20000, 300, 64, 1], [1, 1, 2, 1]),                       # small batch without the sum
    (0, 0, [3000, 700, 5000, 900], [5, 3, 6, 4]),                    # verify rows only
    (0, 0, [2000, 1500, 600, 116], [1, 1, 40, 70]),                  # decodes + prefill, no verify class
    (0, 0, [900, 800], [100, 33]),                                   # prefill rows only
    (128, 0, [6000, 2100, 900, 50], [1, 4, 1, 2]),                   # windowed: one partition each
    (0, 256, [5000, 300, 9000, 40], [1, 1, 5, 2]),                   # the caller's partition
    (0, 0, [33] * 70 + [7000] * 3, [1] * 73),                        # many short ones, few long
])
def test_host_copies_of_the_lengths_plan_the_launches(G, kv_dtype, window, partition, seq_lens,
                                                      q_lens):
    """With args.seq_lens_host / cu_seqlens_q_host the library picks partition sizes, exact
    grids and the kernels that have work on the host.  Same results as without them (and as
    the oracle), for every q_len class mix, including classes without a sequence."""
    b = make_batch(seq_lens, q_lens, window=window, partition=partition, kv_dtype=kv_dtype)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    plain = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, host_lens=True)
    assert_close(out, ref, "host lengths")
    assert_close(plain, ref, "no host lengths, no lse")
    assert np.allclose(lse, ref_lse, atol=2e-3)
    a = synth.bf16_bits_to_f32(out).astype(np.float64)
    # the two ways of planning agree closely on the same kernels (both with lse: the prefill
    # kernel without lse rounds its Q operands once more and may differ by a bf16 ulp)
    plain_lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True)[0]
    c = synth.bf16_bits_to_f32(plain_lse).astype(np.float64)
    assert np.abs(a - c).max() <= 4e-3
    both = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, host_lens=True, hint=True)[0]
    assert np.array_equal(both, out)   # the sum adds nothing the arrays do not say


def test_kernel_events_time_the_split_kv_dispatch(G):
    """eid_debug_set_kernel_events exists in the measurement build only (-DEID_MEASURE): a decode
    call through that build attaches the two events to the split-KV kernel's dispatch; the
    outputs equal the serving library's, the time between the events is a kernel's worth, and
    once switched off the events are left alone.  The serving library has no such symbol."""
    from eidola_amd import _lib
    assert not hasattr(_lib.load_library(), "eid_debug_set_kernel_events")
    lib = _lib.load_measure_library()
    rng = np.random.default_rng(77)
    seq_lens = rng.integers(3000, 9000, size=24)
    b = make_batch(seq_lens, [1] * len(seq_lens), partition=0)
    q, k, v, sinks = logical_tensors(b, seed=9)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    plain = G.run_attn(b, q, kc_d, vc_d, sinks, host_lens=True, hint=True)
    call = ea.prepare("eid_attn_decode", b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table),
                      G.dev(b.seq_lens), max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                      sum_kv_len=int(b.seq_lens.sum()), seq_lens_host=b.seq_lens).bound_to(lib)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    e1.record()
    torch.cuda.synchronize()
    lib.eid_debug_set_kernel_events(e0.cuda_event, e1.cuda_event)
    try:
        timed = G.bits_host(call()).copy()
    finally:
        lib.eid_debug_set_kernel_events(None, None)
    torch.cuda.synchronize()
    assert np.array_equal(timed, plain)
    ms = e0.elapsed_time(e1)
    assert 0.005 < ms < 5.0, ms    # ~0.3 GB of KV: tens of microseconds, not the back-to-back records
    again = G.bits_host(call()).copy()
    torch.cuda.synchronize()
    assert np.array_equal(again, plain) and e0.elapsed_time(e1) == ms


@pytest.mark.parametrize("seed", range(8))
def test_seeded_small_batches_with_long_contexts(G, seed):
    """One to six sequences with contexts drawn log-uniformly up to 20,000 tokens: the
    regime where the host chooses between 512-key partitions with a wave per chunk and the
    split-KV kernel, with and without the sum and the host copies of the lengths."""
    rng = np.random.default_rng(5000 + seed)
    S = int(rng.integers(1, 7))
    q_lens = rng.choice([1, 1, 1, 2, 4, 5, 6], size=S)
    if rng.random() < 0.5:
        q_lens[:] = 1
    top = int(rng.choice([600, 5000, 20000]))
    ctx = np.exp(rng.uniform(0.0, np.log(top), size=S)).astype(np.int64)
    seq_lens = q_lens + ctx
    window = int(rng.choice([0, 0, 0, 128, 2000]))
    kv_dtype = KV_FP8_E4M3 if rng.random() < 0.3 else KV_BF16
    hint, host = bool(rng.random() < 0.5), bool(rng.random() < 0.6)
    b = make_batch(seq_lens, q_lens, window=window, kv_dtype=kv_dtype, seed=seed)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, hint=hint,
                          host_lens=host)
    what = f"seed {seed}: L={seq_lens.tolist()} q={q_lens.tolist()} w={window} dtype={kv_dtype}"
    assert_close(out, ref, what)
    assert np.allclose(lse, ref_lse, atol=3e-3), what


@pytest.mark.parametrize("seed", range(10))
def test_seeded_batches_of_up_to_32_query_rows(G, seed):
    """Query lengths drawn from 1..8, 1..16 or 1..32 in batches of a few to a few dozen
    sequences: the classes that stay on the split-KV kernels with four tiles per wave and
    two or four waves per KV head, or go to the prefill kernel, depending on the batch."""
    rng = np.random.default_rng(9000 + seed)
    S = int(rng.integers(1, int(rng.choice([4, 9, 60]))))
    qmax = int(rng.choice([8, 16, 32]))
    q_lens = rng.integers(1, qmax + 1, size=S)
    top = int(rng.choice([300, 3000, 9000]))
    ctx = np.exp(rng.uniform(0.0, np.log(top), size=S)).astype(np.int64)
    seq_lens = q_lens + ctx
    window = int(rng.choice([0, 0, 0, 128, 1000]))
    partition = int(rng.choice([0, 0, 0, 64, 256, 1024]))
    kv_dtype = KV_FP8_E4M3 if rng.random() < 0.3 else KV_BF16
    hint, host = bool(rng.random() < 0.5), bool(rng.random() < 0.5)
    b = make_batch(seq_lens, q_lens, window=window, partition=partition, kv_dtype=kv_dtype,
                   seed=seed)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True, hint=hint,
                          host_lens=host)
    what = f"seed {seed}: S={S} q<={qmax} w={window} P={partition} dtype={kv_dtype}"
    assert_close(out, ref, what)
    assert np.allclose(lse, ref_lse, atol=3e-3), what
    assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, hint=hint, host_lens=host), ref,
                 what + ", no lse")


# ---------------------------------------------------------------- benchmark configurations
def _sample_check(G, b, q_d, kc_d, vc_d, sinks, out_d, seqs, what, ks=None, vs=None):
    sub, kc, vc = G.compact_to_cpu(b, kc_d, vc_d, seqs)
    rows = G.rows_of(b, seqs)
    qb = G.bits_host(q_d)[rows]
    ref, _ = oracle.attn_f64(desc_of(sub), qb, kc, vc, sub.block_table, sub.seq_lens,
                             sub.cu_seqlens_q, sinks, ks, vs)
    return assert_close(G.bits_host(out_d)[rows], ref, what)


def _gpu_inputs(G, b, pool_seed=7):
    g = b.geom
    dt = torch.uint8 if g.kv_dtype == KV_FP8_E4M3 else torch.bfloat16
    kc_d = torch.empty((b.num_blocks, 16, 8, 64), dtype=dt, device=G.DEV)
    vc_d = torch.empty_like(kc_d)
    ks, vs = synth.fill_pool_gpu(g, kc_d, vc_d, pool_seed)
    q = synth.normal_bf16((b.num_q_tokens, 64, 64), b.seed, synth.TID_Q)
    sinks = synth.bf16_bits_to_f32(synth.normal_bf16((64,), b.seed, synth.TID_SINK))
    return G.bf16_dev(q), kc_d, vc_d, sinks, ks, vs


@pytest.mark.parametrize("window", [0, 128])
def test_config2_full_size(G, window):
    b = synth.config2(window=window)
    assert b.num_seqs == 64 and b.block_table.shape[1] == 512
    q_d, kc_d, vc_d, sinks, _, _ = _gpu_inputs(G, b)
    args = (b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens))
    out = ea.attn_decode(*args, max_kv_len=b.max_kv_len, sinks=G.dev(sinks))
    torch.cuda.synchronize()
    order = np.argsort(b.seq_lens)
    seqs = [int(order[0]), int(order[31]), int(order[-1])] + list(range(4))
    _sample_check(G, b, q_d, kc_d, vc_d, sinks, out, seqs, f"config2 w={window}")
    # size-independent properties: partition size does not matter beyond fp32 round-off
    o = synth.bf16_bits_to_f32(G.bits_host(out))
    assert np.isfinite(o).all()
    for P in (128, 1024):
        g2 = b.with_geom(partition_size=P).geom
        o2 = ea.attn_decode(g2, *args[1:], max_kv_len=b.max_kv_len, sinks=G.dev(sinks))
        torch.cuda.synchronize()
        assert np.abs(synth.bf16_bits_to_f32(G.bits_host(o2)) - o).max() <= 4e-3
        o3 = ea.attn_decode(g2, *args[1:], max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                            sum_kv_len=int(b.seq_lens.sum()))
        torch.cuda.synchronize()
        assert torch.equal(o2, o3)
    # the launch-sizing hint (exact sum, or any upper bound) only trims the grid
    for hint in (int(b.seq_lens.sum()), 2 * int(b.seq_lens.sum()), 64 * b.max_kv_len):
        oh = ea.attn_decode(*args, max_kv_len=b.max_kv_len, sinks=G.dev(sinks), sum_kv_len=hint)
        torch.cuda.synchronize()
        assert torch.equal(oh, out), hint
    # host copy of seq_lens: the library derives on the host the partition the kernels would
    # (the same rule), so the work items and with them every bit of the output are the same
    oh = ea.attn_decode(*args, max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                        sum_kv_len=int(b.seq_lens.sum()), seq_lens_host=b.seq_lens)
    torch.cuda.synchronize()
    assert torch.equal(oh, out)
    # ... and with the host copy of the block table the first chunk's page ids come along
    oh = ea.attn_decode(*args, max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                        seq_lens_host=b.seq_lens, block_table_host=b.block_table)
    torch.cuda.synchronize()
    assert torch.equal(oh, out)


def test_config3_mixed_full_size(G):
    b = synth.config3()
    assert b.num_q_tokens == 4216 and b.num_seqs == 128
    q_d, kc_d, vc_d, sinks, _, _ = _gpu_inputs(G, b)
    # slot-mapped write of every new token precedes attention
    k_new = synth.normal_bf16((4216, 8, 64), b.seed, synth.TID_K)
    v_new = synth.normal_bf16((4216, 8, 64), b.seed, synth.TID_V)
    ea.kv_write(b.geom, G.bf16_dev(k_new), G.bf16_dev(v_new), kc_d, vc_d, G.dev(b.slot_mapping))
    flat = kc_d.view(-1, 8, 64)
    got = G.bits_host(flat[torch.from_numpy(b.slot_mapping).to(G.DEV)])
    assert np.array_equal(got, k_new)
    out = ea.attn_varlen(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                         G.dev(b.cu_seqlens_q), max_q_len=512, max_kv_len=b.max_kv_len,
                         sinks=G.dev(sinks))
    torch.cuda.synchronize()
    assert np.isfinite(synth.bf16_bits_to_f32(G.bits_host(out))).all()
    oh = ea.attn_varlen(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                        G.dev(b.cu_seqlens_q), max_q_len=512, max_kv_len=b.max_kv_len,
                        sinks=G.dev(sinks), sum_kv_len=int(b.seq_lens.sum()))
    torch.cuda.synchronize()
    assert torch.equal(oh, out)
    # all eight prefill chunks (the longest walks 70 chunks of keys) and ten decode rows,
    # among them the shortest and the longest context
    dec = 8 + np.argsort(b.seq_lens[8:])
    seqs = list(range(8)) + [int(dec[0]), int(dec[-1]), int(dec[60])] + [8, 9, 33, 60, 90, 111, 127]
    _sample_check(G, b, q_d, kc_d, vc_d, sinks, out, sorted(set(seqs)), "config3")
    # with the scheduler's host copies of the lengths (the way bench.py calls it): same plan
    # for the prefill rows, host-planned launches for the decode rows
    oh = ea.attn_varlen(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                        G.dev(b.cu_seqlens_q), max_q_len=512, max_kv_len=b.max_kv_len,
                        sinks=G.dev(sinks), sum_kv_len=int(b.seq_lens.sum()),
                        seq_lens_host=b.seq_lens, cu_seqlens_q_host=b.cu_seqlens_q)
    torch.cuda.synchronize()
    _sample_check(G, b, q_d, kc_d, vc_d, sinks, oh, [0, 7, int(dec[-1]), 8, 127], "config3, host lengths")


def test_config2_as_bench_times_it(G):
    """Exactly the call bench.py's headline times, at full size: ONE eid_attn_decode that is
    handed the 64 new K/V rows (fused write), the host copies of seq_lens and the block table
    and their sum, on a page set other than the first of the 300k-block pool.  Sampled
    sequences against the fp64 oracle, and every written cache row bit for bit."""
    b0 = synth.config2()
    nblk = int(((b0.seq_lens.astype(np.int64) + 15) // 16).sum())
    b = synth.config2(perm_offset=3 * nblk)              # page set 3
    assert not np.array_equal(b.block_table, b0.block_table)
    q_d, kc_d, vc_d, sinks, _, _ = _gpu_inputs(G, b)
    k_new = synth.normal_bf16((64, 8, 64), b.seed, synth.TID_K)
    v_new = synth.normal_bf16((64, 8, 64), b.seed, synth.TID_V)
    flat_k, flat_v = kc_d.view(-1, 8, 64), vc_d.view(-1, 8, 64)
    slots = torch.from_numpy(b.slot_mapping).to(G.DEV)
    flat_k[slots] = float("nan")                          # the call has to write these itself
    flat_v[slots] = float("nan")
    out = ea.attn_decode(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                         max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                         sum_kv_len=int(b.seq_lens.sum()), k_new=G.bf16_dev(k_new),
                         v_new=G.bf16_dev(v_new), seq_lens_host=b.seq_lens,
                         block_table_host=b.block_table)
    torch.cuda.synchronize()
    assert np.array_equal(G.bits_host(flat_k[slots]), k_new)
    assert np.array_equal(G.bits_host(flat_v[slots]), v_new)
    order = np.argsort(b.seq_lens)
    seqs = sorted(set([int(order[0]), int(order[1]), int(order[31]), int(order[-1]), int(order[-2])]
                      + list(range(0, 64, 9))))
    _sample_check(G, b, q_d, kc_d, vc_d, sinks, out, seqs, "config2 as bench.py times it")
    # the same call as two launches gives the same bits
    out2 = ea.attn_decode(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                          max_kv_len=b.max_kv_len, sinks=G.dev(sinks))
    torch.cuda.synchronize()
    assert np.abs(synth.bf16_bits_to_f32(G.bits_host(out2)).astype(np.float64)
                  - synth.bf16_bits_to_f32(G.bits_host(out)).astype(np.float64)).max() <= 4e-3


def test_config4_fp8_full_size(G):
    b = synth.config4()
    assert b.num_seqs == 256 and 128 <= b.seq_lens.min() and b.seq_lens.max() <= 32768
    q_d, kc_d, vc_d, sinks, ks, vs = _gpu_inputs(G, b)
    out = ea.attn_decode(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                         max_kv_len=b.max_kv_len, sinks=G.dev(sinks), k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    oh = ea.attn_decode(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                        max_kv_len=b.max_kv_len, sinks=G.dev(sinks), k_scale=ks, v_scale=vs,
                        sum_kv_len=int(b.seq_lens.sum()))
    torch.cuda.synchronize()
    assert torch.equal(oh, out)
    order = np.argsort(b.seq_lens)
    seqs = sorted({int(order[i]) for i in (0, 1, 25, 64, 128, 192, 230, 254, 255)} | {0, 1, 2})
    assert len(seqs) >= 10
    _sample_check(G, b, q_d, kc_d, vc_d, sinks, out, seqs, "config4",
                  ks.cpu().numpy(), vs.cpu().numpy())


@pytest.mark.parametrize("layer", [0, 1])
def test_config5_verify_full_size(G, layer):
    b = synth.config5(layer=layer)
    assert b.num_q_tokens == 640 and b.geom.partition_size == 512
    q_d, kc_d, vc_d, sinks, _, _ = _gpu_inputs(G, b, pool_seed=9 + layer)
    out = ea.attn_varlen(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                         G.dev(b.cu_seqlens_q), max_q_len=5, max_kv_len=b.max_kv_len,
                         sinks=G.dev(sinks))
    torch.cuda.synchronize()
    assert np.isfinite(synth.bf16_bits_to_f32(G.bits_host(out))).all()
    oh = ea.attn_varlen(b.geom, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                        G.dev(b.cu_seqlens_q), max_q_len=5, max_kv_len=b.max_kv_len,
                        sinks=G.dev(sinks), sum_kv_len=int(b.seq_lens.sum()))
    torch.cuda.synchronize()
    assert torch.equal(oh, out)
    # eight sequences: the shortest, the longest, the one nearest to 128 whole partitions of 512
    # keys (the most pieces a row can have), and five spread over the lengths
    order = np.argsort(b.seq_lens)
    most_parts = int(np.argmax((b.seq_lens + 511) // 512 * 100000 - b.seq_lens % 512))
    seqs = sorted({int(order[i]) for i in (0, 16, 40, 64, 90, 112, 127)} | {most_parts})
    assert len(seqs) >= 7 and (b.seq_lens[most_parts] + 511) // 512 == ((b.seq_lens + 511) // 512).max()
    _sample_check(G, b, q_d, kc_d, vc_d, sinks, out, seqs, f"config5 layer {layer}")


def test_step_replayed_from_a_hip_graph(G):
    """kv_write + decode attention captured into a HIP graph and replayed: every replay must
    reproduce the eager result bit for bit, with eager work and synchronisations in between
    (the library enqueues kernels only: no memset nodes, no allocation)."""
    b = make_batch([700, 33, 2500, 129], [1, 1, 1, 1])
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    k_new = G.bf16_dev(synth.normal_bf16((4, 8, 64), 77, synth.TID_K))
    v_new = G.bf16_dev(synth.normal_bf16((4, 8, 64), 77, synth.TID_V))
    slots = G.dev(np.array([b.all_slots(s)[-1] for s in range(4)], dtype=np.int64))
    call = ea.prepare("eid_attn_decode", b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table),
                      G.dev(b.seq_lens), max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                      sum_kv_len=int(b.seq_lens.sum()))

    def step():
        ea.kv_write(b.geom, k_new, v_new, kc_d, vc_d, slots)
        call()

    step()
    torch.cuda.synchronize()
    eager = call.out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for i in range(4):
        call.out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(call.out, eager), f"replay {i}"
        step()                      # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(call.out, eager)


def _mixed_call(G, seed=41):
    """A mixed batch (prefill chunks, verify rows, decodes): its prefill launch runs on the
    library's helper stream beside the split-KV launches."""
    b = make_batch([900, 64, 3000, 200, 1500, 77, 2600], [256, 1, 1, 5, 40, 1, 2], seed=seed)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    call = ea.prepare("eid_attn_varlen", b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table),
                      G.dev(b.seq_lens), G.dev(b.cu_seqlens_q), max_q_len=b.max_q_len,
                      max_kv_len=b.max_kv_len, sinks=G.dev(sinks), sum_kv_len=int(b.seq_lens.sum()))
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    return b, call, ref


def test_mixed_batch_replayed_from_a_hip_graph(G):
    """The fork to the helper stream and the join back are captured with the launches: every
    replay must reproduce the eager result, with eager work in between."""
    b, call, ref = _mixed_call(G)
    call()
    torch.cuda.synchronize()
    eager = call.out.clone()
    assert_close(G.bits_host(eager), ref, "mixed eager")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()                      # the thread's helper stream exists before capture starts
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for i in range(4):
        call.out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(call.out, eager), f"replay {i}"
        call()
        torch.cuda.synchronize()
        assert torch.equal(call.out, eager)


def test_mixed_batches_from_two_host_threads(G):
    """Two host threads, each with its own stream, workspace and output, issue mixed batches at
    the same time: every thread owns its helper stream, results equal the single-threaded ones."""
    import threading
    cases = [_mixed_call(G, seed=51), _mixed_call(G, seed=52)]
    want = []
    for _, call, ref in cases:
        call()
        torch.cuda.synchronize()
        assert_close(G.bits_host(call.out), ref, "mixed single-threaded")
        want.append(call.out.clone())
    errors = []

    def worker(i):
        try:
            torch.cuda.set_device(0)
            st = torch.cuda.Stream()
            _, call, _ = cases[i]
            for it in range(20):
                call.out.zero_()            # on the default stream of this thread ...
                st.wait_stream(torch.cuda.current_stream())
                call(stream=st.cuda_stream)
                st.synchronize()
                if not torch.equal(call.out, want[i]):
                    errors.append((i, it))
                    return
        except Exception as ex:  # surfaced below
            errors.append((i, repr(ex)))

    ts = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("window", [0, 700])
def test_prefill_key_range_split(G, kv_dtype, window):
    """Few query tiles over long contexts: the prefill kernel splits every tile's key range into
    parts (here 8, 4 and 2 by the planning rule) that are merged afterwards.  Covered: a chunk
    whose context is shorter than one part (empty parts), chunks without prior context, decode
    and verify rows in the same batch (their tokens must be left alone by the merge), fp8."""
    cases = [
        ([5200], [200]),                                   # 8 parts
        ([3000, 140, 40, 2600], [100, 100, 40, 7]),         # short contexts beside long ones
        ([4000, 900, 2500, 64, 1800], [64, 1, 5, 64, 2]),   # mixed classes
    ]
    for seq_lens, q_lens in cases:
        b = make_batch(seq_lens, q_lens, seed=43, window=window, kv_dtype=kv_dtype)
        q, k, v, sinks = logical_tensors(b)
        ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
        kc, vc = cpu_caches(b, k, v, ks, vs)
        kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
        ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
        out, lse = G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, return_lse=True)
        assert_close(out, ref, f"split prefill {seq_lens} w={window}")
        assert np.allclose(lse, ref_lse, atol=2e-3)
        assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs), ref,
                     f"split prefill {seq_lens} w={window}, no lse")


def test_large_values_across_several_partitions(G):
    """Split-KV partials carry a partition's normalised output in fp16.  Values of a few
    ten thousand are exact to fp16 relative precision; beyond 65,504 (which bf16 holds) a
    sequence cut into several pieces saturates instead of going to inf / NaN, and a sequence
    that stays in one piece is not affected at all."""
    seq_lens, q_lens = [3000, 1500, 200], [1, 1, 1]
    for scale, exact in ((3.0e4, True), (1.0e5, False)):
        b = make_batch(seq_lens, q_lens, partition=256)
        q, k, v, sinks = logical_tensors(b, seed=31)
        # values uniform in [-scale, scale], exactly representable pattern: bf16 of N(0,1) * scale / 4
        vf = np.clip(synth.bf16_bits_to_f32(v) * (scale / 4), -scale, scale).astype(np.float32)
        v = synth.f32_to_bf16_bits(vf)
        kc, vc = cpu_caches(b, k, v)
        kc_d, vc_d = G.gpu_caches(b, k, v)
        ref, _ = oracle_out(b, q, kc, vc, sinks)
        got = synth.bf16_bits_to_f32(G.run_attn(b, q, kc_d, vc_d, sinks)).astype(np.float64)
        assert np.isfinite(got).all()
        err = np.abs(got - ref)
        rows = b.cu_seqlens_q
        if exact:   # the usual tolerance, relative to the magnitude of the values
            assert err.max() <= MAX_ABS_TOL_REL * scale and err.mean() <= MEAN_ABS_TOL_REL * scale
        else:       # bounded, never NaN; the single-piece sequence (200 keys) is exact
            assert err.max() <= scale
            one = slice(rows[2], rows[3])
            assert err[one].max() <= MAX_ABS_TOL_REL * scale


def test_a_partial_per_partition_when_asked_for():
    """EID_STORE_EVERY_PARTITION=1 (a measurement aid read once per process) makes an even
    split store every partition of the caller's size and leaves all merging to the merge
    kernel; checked in a process of its own against the oracle, on a verify batch large enough
    for the even split."""
    import os
    import subprocess
    import sys
    code = r'''
import numpy as np, torch, sys, os
sys.path.insert(0, os.path.join(os.getcwd(), "tests"))
import gpu_helpers as G
from helpers import make_batch, logical_tensors, cpu_caches, oracle_out, assert_close
rng = np.random.default_rng(5)
seq_lens = rng.integers(1500, 9000, size=40)
b = make_batch(seq_lens, [5] * 40, partition=128)
q, k, v, sinks = logical_tensors(b)
kc, vc = cpu_caches(b, k, v)
kc_d, vc_d = G.gpu_caches(b, k, v)
ref, _ = oracle_out(b, q, kc, vc, sinks)
for host in (False, True):
    print(assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, host_lens=host, hint=host), ref, "every partition"))
# decode rows over an fp8 cache (two KV heads per wave, raw bytes through LDS), 128-key partitions
from eidola_amd import KV_FP8_E4M3
from helpers import fp8_scales
seq_lens = rng.integers(2500, 6000, size=48)
b = make_batch(seq_lens, [1] * 48, partition=128, kv_dtype=KV_FP8_E4M3)
q, k, v, sinks = logical_tensors(b)
ks, vs = fp8_scales(k, v)
kc, vc = cpu_caches(b, k, v, ks, vs)
kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
ref, _ = oracle_out(b, q, kc, vc, sinks, ks, vs)
for host in (False, True):
    print(assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, host_lens=host, hint=host), ref, "every partition, fp8"))
# verify rows over an fp8 cache (one KV head per wave, raw bytes through LDS)
seq_lens = rng.integers(1500, 7000, size=40)
b = make_batch(seq_lens, [4, 6] * 20, partition=128, kv_dtype=KV_FP8_E4M3)
q, k, v, sinks = logical_tensors(b)
ks, vs = fp8_scales(k, v)
kc, vc = cpu_caches(b, k, v, ks, vs)
kc_d, vc_d = G.gpu_caches(b, k, v, ks, vs)
ref, _ = oracle_out(b, q, kc, vc, sinks, ks, vs)
for host in (False, True):
    print(assert_close(G.run_attn(b, q, kc_d, vc_d, sinks, ks, vs, host_lens=host, hint=host), ref, "every partition, fp8 verify"))
'''
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, EID_STORE_EVERY_PARTITION="1")
    r = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
