"""Pins the CPU oracle (oracle/eid_oracle.c) without any reference implementation:
closed forms of softmax-with-sink, a library routine for the sink = -inf case, an
independent numpy restatement on brute-force-sized inputs, and the invariances the
definition implies (window >= context, page permutation, partition size)."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import oracle_np
from eidola_amd import KV_BF16, KV_FP8_E4M3, synth

from helpers import (make_batch, desc_of, logical_tensors, cpu_caches, oracle_out, fp8_scales,
                     all_slots, empty_caches)


def bits(x):
    return synth.f32_to_bf16_bits(np.asarray(x, dtype=np.float32))


def f(x):
    return synth.bf16_bits_to_f32(x).astype(np.float64)


# ---------------------------------------------------------------- scalar conversions
def test_bf16_roundtrip_and_rne():
    L = oracle.lib()
    # every bf16 pattern survives widen -> narrow
    for h in list(range(0, 0x7F80, 97)) + [0x0000, 0x8000, 0x7F7F, 0x0001, 0x3F80]:
        assert L.orc_f32_to_bf16(L.orc_bf16_to_f32(h)) == h
    # ties to even: 1 + 2^-8 is halfway between 1.0 (even) and 1 + 2^-7
    assert L.orc_f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    assert L.orc_f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82
    # numpy mirror agrees on random values
    x = np.random.default_rng(0).standard_normal(5000).astype(np.float32)
    assert all(L.orc_f32_to_bf16(float(v)) == int(b) for v, b in zip(x, synth.f32_to_bf16_bits(x)))


def test_fp8_decode_matches_format_definition_and_torch():
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.fp8_decode(codes).astype(np.float64)
    want = oracle_np.fp8_e4m3_to_f64(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    t = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy().astype(np.float64)
    ok = ~np.isnan(want)
    assert np.array_equal(t[ok], want[ok])
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9


def test_fp8_encode_known_answers():
    enc = oracle.lib().orc_fp8_e4m3_encode
    assert enc(0.0) == 0x00 and enc(-0.0) == 0x80
    assert enc(448.0) == 0x7E and enc(1e9) == 0x7E and enc(-1e9) == 0xFE
    assert enc(float("inf")) == 0x7E and enc(float("nan")) == 0x7F
    assert enc(464.0) == 0x7E and enc(465.0) == 0x7E      # saturates where torch gives NaN
    assert enc(1.0) == 0x38 and enc(1.0625) == 0x38       # tie -> even mantissa (1.0)
    assert enc(1.1875) == 0x3A                            # tie between 1.125 and 1.25 -> 1.25
    assert enc(2.0 ** -10) == 0x00                        # half the smallest subnormal: tie -> 0
    assert enc(1.5 * 2.0 ** -9) == 0x02                   # tie between 1 and 2 subnormal steps
    assert enc(7.5 * 2.0 ** -9) == 0x08                   # rounds up into the smallest normal
    assert enc(1e-4) == 0x00


def test_fp8_encode_exhaustive_over_bf16_against_search_encoder():
    """ALL finite bf16 inputs (the only values kv_write ever quantises, 65,280 of them) against
    the exhaustive-search encoder; their quotients by three other scales on a stride."""
    all_bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = synth.bf16_bits_to_f32(all_bits)
    xs = x[np.isfinite(x)]
    assert len(xs) == 65280
    got = oracle.fp8_encode(xs)
    want = oracle_np.fp8_e4m3_encode_np(xs)
    assert np.array_equal(got, want)
    # in-range agreement with torch's converter (which does not saturate beyond 448+)
    inr = np.abs(xs) <= 448
    t = torch.from_numpy(xs[inr].copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got[inr], t)
    for scale in (np.float32(0.0078125), np.float32(0.0123), np.float32(3.7)):
        ys = (xs[::13] / scale).astype(np.float32)          # IEEE fp32 division, as kv_write does
        assert np.array_equal(oracle.fp8_encode(ys), oracle_np.fp8_e4m3_encode_np(ys))


# ---------------------------------------------------------------- K1
def test_kv_write_roundtrip_skips_and_poison():
    b = make_batch([37, 5, 64], [1, 1, 1])
    q, k, v, _ = logical_tensors(b)
    kc, vc = empty_caches(b)
    slots = all_slots(b)
    sm = slots.copy()
    sm[3] = -1                                            # padding row: must be skipped
    oracle.kv_write(desc_of(b), k, v, kc, vc, sm)
    kf = kc.reshape(-1, 8, 64)
    vf = vc.reshape(-1, 8, 64)
    keep = np.ones(len(slots), bool)
    keep[3] = False
    assert np.array_equal(kf[slots[keep]], k[keep]) and np.array_equal(vf[slots[keep]], v[keep])
    untouched = np.ones(kf.shape[0], bool)
    untouched[slots[keep]] = False
    assert (kf[untouched] == 0x7FC1).all() and (vf[untouched] == 0x7FC1).all()
    with pytest.raises(ValueError):
        oracle.kv_write(desc_of(b), k[:1], v[:1], kc, vc, np.array([b.num_blocks * 16]))


def test_kv_write_fp8_matches_definition():
    b = make_batch([50], [1], kv_dtype=KV_FP8_E4M3)
    q, k, v, _ = logical_tensors(b)
    ks, vs = fp8_scales(k, v)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    slots = all_slots(b)
    x = synth.bf16_bits_to_f32(k) / ks[None, :, None]     # fp32 IEEE division
    want = oracle_np.fp8_e4m3_encode_np(x[:6])
    assert np.array_equal(kc.reshape(-1, 8, 64)[slots[:6]], want)
    # absmax element lands exactly on +-448
    assert (np.abs(oracle_np.fp8_e4m3_to_f64(kc.reshape(-1, 8, 64)[slots])).max(axis=(0, 2)) == 448).all()


# ---------------------------------------------------------------- closed forms
def _single_seq(L, q_len=1, window=0, seed=3):
    b = make_batch([L], [q_len], window=window, seed=seed)
    q, k, v, sinks = logical_tensors(b)
    return b, q, k, v, sinks


def test_closed_form_constant_v():
    """All V rows equal c  =>  out = c * (1 - p_sink), p_sink = e^(sink-m)/den."""
    b, q, k, v, sinks = _single_seq(40)
    c = synth.normal_bf16((8, 64), 99, 1)
    v[:] = c[None]
    kc, vc = cpu_caches(b, k, v)
    out, lse = oracle_out(b, q, kc, vc, sinks)
    s = 0.125 * np.einsum("hd,lhd->hl", f(q[0]).reshape(8, 8, 64).reshape(64, 64),
                          np.repeat(f(k), 8, axis=1))
    for h in range(64):
        p_sink = math.exp(float(sinks[h]) - lse[0, h])
        assert np.allclose(out[0, h], f(c[h // 8]) * (1 - p_sink), rtol=1e-12, atol=1e-14)
        assert np.isclose(lse[0, h], np.log(np.exp(s[h]).sum() + math.exp(float(sinks[h]))), rtol=1e-12)


def test_closed_form_single_key_is_sigmoid():
    """One key  =>  out = v0 * sigmoid(s0 - sink)."""
    b, q, k, v, sinks = _single_seq(1)
    kc, vc = cpu_caches(b, k, v)
    out, _ = oracle_out(b, q, kc, vc, sinks)
    for h in range(64):
        s0 = 0.125 * float(f(q[0, h]) @ f(k[0, h // 8]))
        sig = 1.0 / (1.0 + math.exp(float(sinks[h]) - s0))
        assert np.allclose(out[0, h], f(v[0, h // 8]) * sig, rtol=1e-12, atol=1e-15)


def test_closed_form_zero_query_is_damped_mean():
    """Q = 0  =>  out = mean(V_allowed) * n / (n + e^sink)."""
    b, q, k, v, sinks = _single_seq(33)
    q[:] = 0
    kc, vc = cpu_caches(b, k, v)
    out, _ = oracle_out(b, q, kc, vc, sinks)
    n = 33
    for h in range(0, 64, 5):
        want = f(v[:, h // 8]).mean(axis=0) * n / (n + math.exp(float(sinks[h])))
        assert np.allclose(out[0, h], want, rtol=1e-12, atol=1e-15)


def test_large_sink_drives_output_to_zero_and_no_sink_is_plain_softmax():
    b, q, k, v, sinks = _single_seq(20)
    kc, vc = cpu_caches(b, k, v)
    big = np.full(64, 80.0, np.float32)
    out, _ = oracle_out(b, q, kc, vc, big)
    assert np.abs(out).max() < 1e-25
    out_ns, _ = oracle_out(b, q, kc, vc, None)
    tiny = np.full(64, -80.0, np.float32)
    out_t, _ = oracle_out(b, q, kc, vc, tiny)
    assert np.allclose(out_ns, out_t, rtol=1e-12, atol=1e-30)


def test_sink_counted_once_independent_of_context_split():
    """den must contain e^sink exactly once: compare with the explicit formula."""
    b, q, k, v, sinks = _single_seq(600)
    kc, vc = cpu_caches(b, k, v)
    _, lse = oracle_out(b, q, kc, vc, sinks)
    for h in (0, 17, 63):
        s = 0.125 * f(k[:, h // 8]) @ f(q[0, h])
        assert np.isclose(math.exp(lse[0, h]), np.exp(s).sum() + math.exp(float(sinks[h])), rtol=1e-11)


# ---------------------------------------------------------------- library routine
@pytest.mark.parametrize("L,q_len", [(37, 1), (64, 5), (100, 100), (300, 64)])
def test_matches_torch_sdpa_when_sink_is_minus_inf(L, q_len):
    b, q, k, v, _ = _single_seq(L, q_len)
    kc, vc = cpu_caches(b, k, v)
    out, _ = oracle_out(b, q, kc, vc, None)
    qt = torch.from_numpy(f(q)).permute(1, 0, 2)[None]                     # [1,Hq,q,D]
    kt = torch.from_numpy(np.repeat(f(k), 8, axis=1)).permute(1, 0, 2)[None]
    vt = torch.from_numpy(np.repeat(f(v), 8, axis=1)).permute(1, 0, 2)[None]
    mask = torch.tril(torch.ones(q_len, L, dtype=torch.bool), diagonal=L - q_len)
    ref = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=mask, scale=0.125)
    assert np.allclose(out, ref[0].permute(1, 0, 2).numpy(), rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------- independent restatement
@pytest.mark.parametrize("window", [0, 1, 7, 128])
@pytest.mark.parametrize("fp8", [False, True])
def test_matches_numpy_restatement_on_ragged_batches(window, fp8):
    seq_lens, q_lens = [1, 17, 40, 133, 16], [1, 3, 40, 5, 1]
    b = make_batch(seq_lens, q_lens, window=window, kv_dtype=KV_FP8_E4M3 if fp8 else KV_BF16)
    q, k, v, sinks = logical_tensors(b)
    ks, vs = fp8_scales(k, v) if fp8 else (None, None)
    kc, vc = cpu_caches(b, k, v, ks, vs)
    out, lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
    ref, ref_lse = oracle_np.attention(q, kc, vc, b.block_table, b.seq_lens, b.q_lens,
                                       num_kv_heads=8, scale=0.125, window=window, sinks=sinks,
                                       fp8=fp8, k_scale=ks, v_scale=vs)
    assert np.allclose(out, ref, rtol=1e-10, atol=1e-13)
    assert np.allclose(lse, ref_lse, rtol=1e-12)


def test_non_default_head_count():
    b = make_batch([23, 70], [1, 4], num_kv_heads=2)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    out, _ = oracle_out(b, q, kc, vc, sinks)
    ref, _ = oracle_np.attention(q, kc, vc, b.block_table, b.seq_lens, b.q_lens, num_kv_heads=2,
                                 scale=0.125, sinks=sinks)
    assert np.allclose(out, ref, rtol=1e-10, atol=1e-13)


# ---------------------------------------------------------------- invariances
def test_window_at_least_context_equals_full_bit_for_bit_and_window_one_is_self_only():
    seq_lens, q_lens = [90, 31], [4, 1]
    b0 = make_batch(seq_lens, q_lens, window=0)
    q, k, v, sinks = logical_tensors(b0)
    kc, vc = cpu_caches(b0, k, v)
    full, _ = oracle_out(b0, q, kc, vc, sinks)
    wide, _ = oracle_out(b0.with_geom(window=90), q, kc, vc, sinks)
    assert np.array_equal(full, wide)
    one, _ = oracle_out(b0.with_geom(window=1), q, kc, vc, sinks)
    # row 0 of sequence 0 sits at position 86 and sees only key 86
    h = 9
    s0 = 0.125 * float(f(q[0, h]) @ f(k[86, h // 8]))
    assert np.allclose(one[0, h], f(v[86, h // 8]) / (1 + math.exp(float(sinks[h]) - s0)), rtol=1e-12)


def test_page_permutation_and_pool_size_do_not_change_results():
    seq_lens, q_lens = [200, 45, 16], [1, 5, 1]
    a = make_batch(seq_lens, q_lens, seed=11)
    q, k, v, sinks = logical_tensors(a, seed=5)
    ka, va = cpu_caches(a, k, v)
    ref, _ = oracle_out(a, q, ka, va, sinks)
    for other in (make_batch(seq_lens, q_lens, seed=12, num_blocks=97),
                  make_batch(seq_lens, q_lens, shuffle=False)):
        kb, vb = cpu_caches(other, k, v)
        got, _ = oracle_out(other, q, kb, vb, sinks)
        assert np.array_equal(ref, got)


def test_batch_neighbours_do_not_matter():
    a = make_batch([70, 33, 129], [2, 1, 5])
    q, k, v, sinks = logical_tensors(a)
    kc, vc = cpu_caches(a, k, v)
    ref, _ = oracle_out(a, q, kc, vc, sinks)
    solo = make_batch([33], [1])
    ks, vs = k[70:103], v[70:103]
    kc1, vc1 = cpu_caches(solo, ks, vs)
    got, _ = oracle_out(solo, q[2:3], kc1, vc1, sinks)
    assert np.array_equal(ref[2:3], got)


@pytest.mark.parametrize("window", [0, 64])
def test_splitkv_merge_independent_of_partition_size(window):
    seq_lens, q_lens = [700, 65, 1], [5, 1, 1]
    b = make_batch(seq_lens, q_lens, window=window)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    ref, ref_lse = oracle_out(b, q, kc, vc, sinks)
    d = desc_of(b)
    for P in (64, 128, 512, 4096):
        span = max(int(L) - oracle.lib().orc_kv_begin(int(L), int(ql), window, 16)
                   for L, ql in zip(seq_lens, q_lens))
        nparts = (span + P - 1) // P + 1          # one deliberately empty partition at the end
        ml, acc = oracle.splitkv_f64(d, P, nparts, q, kc, vc, b.block_table, b.seq_lens,
                                     b.cu_seqlens_q)
        assert (ml[..., -1, 1] == 0).all() and np.isneginf(ml[..., -1, 0]).all()
        out, lse = oracle.lse_merge_f64(ml, acc, sinks)
        assert np.isfinite(out).all()
        assert np.allclose(out, ref, rtol=1e-11, atol=1e-14)
        assert np.allclose(lse, ref_lse, rtol=1e-12)


def test_verify_row_equals_decode_at_shorter_context():
    """Row t of a 5-row verify at context L equals a decode at context L - 4 + t."""
    L = 150
    b5 = make_batch([L], [5])
    q, k, v, sinks = logical_tensors(b5)
    kc, vc = cpu_caches(b5, k, v)
    out5, _ = oracle_out(b5, q, kc, vc, sinks)
    for t in range(5):
        b1 = make_batch([L - 4 + t], [1])
        kc1, vc1 = cpu_caches(b1, k[:L - 4 + t], v[:L - 4 + t])
        out1, _ = oracle_out(b1, q[t:t + 1], kc1, vc1, sinks)
        assert np.allclose(out5[t], out1[0], rtol=1e-13, atol=1e-16)


def test_cpu_baseline_path_within_tolerance_of_fp64():
    from helpers import assert_close
    for window, fp8 in ((0, False), (16, False), (0, True)):
        b = make_batch([300, 17, 64], [5, 1, 20], window=window,
                       kv_dtype=KV_FP8_E4M3 if fp8 else KV_BF16)
        q, k, v, sinks = logical_tensors(b)
        ks, vs = fp8_scales(k, v) if fp8 else (None, None)
        kc, vc = cpu_caches(b, k, v, ks, vs)
        ref, ref_lse = oracle_out(b, q, kc, vc, sinks, ks, vs)
        got, lse = oracle.attn_bf16(desc_of(b), q, kc, vc, b.block_table, b.seq_lens,
                                    b.cu_seqlens_q, sinks, ks, vs)
        assert_close(got, ref, f"cpu baseline w={window} fp8={fp8}")
        assert np.allclose(lse, ref_lse, atol=1e-4)
