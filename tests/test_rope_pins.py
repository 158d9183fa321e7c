"""Pins for the oracle of the fused RoPE + QKV split + KV write (orc_rope_kv_write) and for
the YaRN table helper.  The reference holds no model code, so parity with it is unpinned;
what pins the oracle: the identity rotation, an exact numpy emulation of the stated fp32
arithmetic, an independently structured complex-number restatement in fp64, norm and
relative-position invariants of a rotation, and composition with the KV-write rule."""
import numpy as np
import pytest

import oracle
import eidola_amd as ea
from eidola_amd import KV_BF16, KV_FP8_E4M3, synth

HQ, HKV, D = 64, 8, 64


def _desc(kv_dtype=KV_BF16, nb=8, hkv=HKV):
    g = ea.AttnGeometry(num_q_heads=8 * hkv, num_kv_heads=hkv, kv_dtype=kv_dtype)
    return ea.make_desc(g, num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                        max_blocks_per_seq=1, num_blocks=nb)


def _inputs(T, seed, max_pos, hkv=HKV):
    rng = np.random.default_rng(seed)
    qkv = synth.normal_bf16((T, (10 * hkv) * D), seed, synth.TID_Q)
    pos = rng.integers(0, max_pos, size=T).astype(np.int32)
    slots = rng.permutation(8 * 16)[:T].astype(np.int64)
    return qkv, pos, slots


def _f32(bits):
    return synth.bf16_bits_to_f32(bits)


def _to_bf16_rne(x32):
    u = np.asarray(x32, np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def test_identity_table_moves_bits_unchanged():
    T = 20
    qkv, pos, slots = _inputs(T, 1, 4)
    table = np.concatenate([np.ones((4, 32)), np.zeros((4, 32))], axis=1).astype(np.float32)
    kc = np.full((8, 16, HKV, D), 0xABCD, np.uint16)
    vc = np.full((8, 16, HKV, D), 0xABCD, np.uint16)
    slots[::5] = -1
    q = oracle.rope_kv_write(_desc(), qkv, pos, table, kc, vc, slots)
    rows = qkv.reshape(T, 10 * HKV, D)
    assert np.array_equal(q, rows[:, :HQ])
    flat_k, flat_v = kc.reshape(-1, HKV, D), vc.reshape(-1, HKV, D)
    for t in range(T):
        if slots[t] >= 0:
            assert np.array_equal(flat_k[slots[t]], rows[t, HQ:HQ + HKV])
            assert np.array_equal(flat_v[slots[t]], rows[t, HQ + HKV:])
    untouched = np.setdiff1d(np.arange(128), slots[slots >= 0])
    assert (flat_k[untouched] == 0xABCD).all() and (flat_v[untouched] == 0xABCD).all()


@pytest.mark.parametrize("scaling", [1.0, 32.0])
def test_against_exact_emulation_and_complex_restatement(scaling):
    T, max_pos = 64, 5000
    qkv, pos, slots = _inputs(T, 2, max_pos)
    table = ea.yarn_cos_sin(max_pos, scaling_factor=scaling)
    kc = np.zeros((8, 16, HKV, D), np.uint16)
    vc = np.zeros((8, 16, HKV, D), np.uint16)
    q = oracle.rope_kv_write(_desc(), qkv, pos, table, kc, vc, slots)
    rows = qkv.reshape(T, 10 * HKV, D)
    x = _f32(rows[:, :HQ + HKV])                       # rotated heads
    x1, x2 = x[..., :32], x[..., 32:]
    c, s = table[pos][:, None, :32], table[pos][:, None, 32:]
    # (a) the stated arithmetic, emulated: fp32 product, then a fused multiply-add whose exact
    # value fits fp64 (24-bit x 24-bit product plus a 24-bit addend)
    p1, p2 = (x1 * c).astype(np.float32), (x2 * c).astype(np.float32)
    o1 = (-(x2.astype(np.float64)) * s.astype(np.float64) + p1.astype(np.float64)).astype(np.float32)
    o2 = (x1.astype(np.float64) * s.astype(np.float64) + p2.astype(np.float64)).astype(np.float32)
    emu = _to_bf16_rne(np.concatenate([o1, o2], axis=-1))
    got = np.concatenate([q, kc.reshape(-1, HKV, D)[slots]], axis=1)
    assert np.array_equal(got, emu)
    # (b) a differently structured restatement: complex multiplication in fp64.  It differs
    # from the fp32 path by at most one bf16 step on the rare values that sit on a tie.
    z = (x1.astype(np.float64) + 1j * x2.astype(np.float64)) * (c.astype(np.float64) + 1j * s.astype(np.float64))
    ref = np.concatenate([z.real, z.imag], axis=-1)
    err = np.abs(_f32(got).astype(np.float64) - ref)
    mag = (np.abs(x1) + np.abs(x2)).astype(np.float64) * (np.abs(c) + np.abs(s))
    mag = np.concatenate([mag, mag], axis=-1)          # fp32 rounding scales with the operands
    assert (err <= np.abs(ref) * 2.0 ** -8 + mag * 2.0 ** -21).all()
    assert (got != _to_bf16_rne(ref.astype(np.float32))).mean() < 2e-3
    # V is moved, not rotated
    assert np.array_equal(vc.reshape(-1, HKV, D)[slots], rows[:, HQ + HKV:])


def test_rotation_invariants():
    """A rotation keeps norms (times the temperature factor) and makes <q_p, k_r> a function
    of p - r only."""
    max_pos = 3000
    table = ea.yarn_cos_sin(max_pos, scaling_factor=32.0)
    conc = 0.1 * np.log(32.0) + 1.0
    rng = np.random.default_rng(4)
    base = synth.normal_bf16((1, 10 * HKV * D), 9, synth.TID_K)
    T = 40
    qkv = np.repeat(base, T, axis=0)                   # the same vectors at many positions
    pos = np.concatenate([np.arange(0, 20), np.arange(1000, 1020)]).astype(np.int32)
    slots = np.arange(T, dtype=np.int64)
    kc = np.zeros((8, 16, HKV, D), np.uint16)
    vc = np.zeros_like(kc)
    q = _f32(oracle.rope_kv_write(_desc(), qkv, pos, table, kc, vc, slots)).astype(np.float64)
    k = _f32(kc.reshape(-1, HKV, D)[:T]).astype(np.float64)
    x = _f32(base.reshape(10 * HKV, D)).astype(np.float64)
    assert np.allclose((q ** 2).sum(-1), conc ** 2 * (x[:HQ] ** 2).sum(-1)[None], rtol=2e-2)
    # same offset (7) at two absolute positions: p=10,r=3 and p=1010,r=1003
    d1 = (q[10, :8] * k[3, 0]).sum(-1)
    d2 = (q[30, :8] * k[23, 0]).sum(-1)
    assert np.allclose(d1, d2, atol=0.15 * conc ** 2)
    # and it does depend on the offset
    d3 = (q[10, :8] * k[9, 0]).sum(-1)
    assert np.abs(d1 - d3).max() > 1.0


def test_fp8_equals_rotation_then_kv_write():
    T, max_pos = 48, 600
    qkv, pos, slots = _inputs(T, 6, max_pos)
    table = ea.yarn_cos_sin(max_pos)
    ks = np.linspace(0.01, 0.02, HKV).astype(np.float32)
    vs = np.linspace(0.02, 0.01, HKV).astype(np.float32)
    kb = np.zeros((8, 16, HKV, D), np.uint16)
    vb = np.zeros_like(kb)
    q_b = oracle.rope_kv_write(_desc(), qkv, pos, table, kb, vb, slots)
    k8 = np.full((8, 16, HKV, D), 0x5A, np.uint8)
    v8 = np.full_like(k8, 0x5A)
    q_8 = oracle.rope_kv_write(_desc(KV_FP8_E4M3), qkv, pos, table, k8, v8, slots, ks, vs)
    assert np.array_equal(q_b, q_8)
    k8b = np.full_like(k8, 0x5A)
    v8b = np.full_like(k8, 0x5A)
    oracle.kv_write(_desc(KV_FP8_E4M3), kb.reshape(-1, HKV, D)[slots], vb.reshape(-1, HKV, D)[slots],
                    k8b, v8b, slots, ks, vs)
    assert np.array_equal(k8, k8b) and np.array_equal(v8, v8b)


def test_positions_outside_the_table_are_clamped():
    qkv, _, slots = _inputs(4, 7, 10)
    table = ea.yarn_cos_sin(10)
    kc = np.zeros((8, 16, HKV, D), np.uint16)
    vc = np.zeros_like(kc)
    a = oracle.rope_kv_write(_desc(), qkv, np.array([-3, 0, 9, 500], np.int32), table, kc, vc, slots)
    b = oracle.rope_kv_write(_desc(), qkv, np.array([0, 0, 9, 9], np.int32), table, kc.copy(), vc.copy(), slots)
    assert np.array_equal(a, b)


def test_yarn_table_shape_and_limits():
    t = ea.yarn_cos_sin(64, scaling_factor=1.0)
    ang = np.arange(64)[:, None] / (150000.0 ** (np.arange(0, 64, 2) / 64.0))[None]
    assert t.shape == (64, 64) and t.dtype == np.float32
    assert np.allclose(t[:, :32], np.cos(ang), atol=1e-6) and np.allclose(t[:, 32:], np.sin(ang), atol=1e-6)
    y = ea.yarn_cos_sin(64)
    conc = 0.1 * np.log(32.0) + 1.0
    assert np.allclose(y[0, :32], conc) and np.allclose(y[0, 32:], 0.0)
    # the fastest dimension is extrapolated (plain frequency 1), the slowest interpolated (/32)
    assert np.allclose(y[:, 0], conc * np.cos(np.arange(64)), atol=1e-5)
    slow = 1.0 / (32.0 * 150000.0 ** (62.0 / 64.0))
    assert np.allclose(y[:, 63], conc * np.sin(np.arange(64) * slow), atol=1e-6)
