"""GPU parity of eid_rope_kv_write against the CPU oracle: bit-exact (the arithmetic is
fixed: fp32 product, fused multiply-add, bf16 round-to-nearest-even), bf16 and fp8 caches,
skipped slots, poison canaries, other KV-head counts, clamped positions, and the whole
front of a step (fused rotation + write, then attention) against rotation-then-oracle."""
import numpy as np
import pytest
import torch

import oracle
import eidola_amd as ea
from eidola_amd import KV_BF16, KV_FP8_E4M3, _lib, synth

from helpers import assert_close

pytestmark = pytest.mark.gpu
D = 64


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


def _case(T, hkv, kv_dtype, nb, seed, max_pos):
    g = ea.AttnGeometry(num_q_heads=8 * hkv, num_kv_heads=hkv, kv_dtype=kv_dtype)
    desc = ea.make_desc(g, num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                        max_blocks_per_seq=1, num_blocks=nb)
    rng = np.random.default_rng(seed)
    qkv = synth.normal_bf16((T, 10 * hkv * D), seed, synth.TID_Q)
    pos = rng.integers(0, max_pos, size=T).astype(np.int32)
    slots = rng.permutation(nb * 16)[:T].astype(np.int64)
    slots[::7] = -1
    return g, desc, qkv, pos, slots


@pytest.mark.parametrize("hkv", [1, 8, 16])
@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
def test_bit_exact_against_the_oracle(G, hkv, kv_dtype):
    T, nb, max_pos = 333, 40, 6000
    g, desc, qkv, pos, slots = _case(T, hkv, kv_dtype, nb, 21 + hkv, max_pos)
    pos[:3] = [-5, max_pos + 17, max_pos - 1]          # clamped into the table
    table = ea.yarn_cos_sin(max_pos)
    if kv_dtype == KV_FP8_E4M3:
        fill, dt = 0x5A, np.uint8
        ks = np.linspace(0.008, 0.02, hkv).astype(np.float32)
        vs = np.linspace(0.02, 0.008, hkv).astype(np.float32)
    else:
        fill, dt, ks, vs = 0xABCD, np.uint16, None, None
    kc = np.full((nb, 16, hkv, D), fill, dt)
    vc = np.full((nb, 16, hkv, D), fill, dt)
    kc_d, vc_d = G.cache_dev(kc.copy()), G.cache_dev(vc.copy())
    q_ref = oracle.rope_kv_write(desc, qkv, pos, table, kc, vc, slots, ks, vs)
    q_d = ea.rope_kv_write(g, G.bf16_dev(qkv), G.dev(pos), G.dev(table), kc_d, vc_d, G.dev(slots),
                           G.dev(ks), G.dev(vs))
    torch.cuda.synchronize()
    assert np.array_equal(G.bits_host(q_d), q_ref)
    assert np.array_equal(G.cache_host(kc_d), kc) and np.array_equal(G.cache_host(vc_d), vc)


def test_empty_and_argument_errors(G):
    g = ea.AttnGeometry()
    kc = torch.zeros((4, 16, 8, 64), dtype=torch.bfloat16, device=G.DEV)
    table = G.dev(ea.yarn_cos_sin(16))
    q = ea.rope_kv_write(g, torch.empty((0, 5120), dtype=torch.bfloat16, device=G.DEV),
                         torch.empty(0, dtype=torch.int32, device=G.DEV), table, kc, kc.clone(),
                         torch.empty(0, dtype=torch.int64, device=G.DEV))
    assert q.shape == (0, 64, 64)
    with pytest.raises(ValueError):
        ea.rope_kv_write(g, torch.empty((2, 100), dtype=torch.bfloat16, device=G.DEV),
                         torch.zeros(2, dtype=torch.int32, device=G.DEV), table, kc, kc.clone(),
                         torch.zeros(2, dtype=torch.int64, device=G.DEV))


def test_front_of_a_step_then_attention(G):
    """Projection output -> fused rotation + write -> decode attention, against the oracle fed
    with the oracle's own rotation: the pieces compose."""
    hkv, nb, max_pos = 8, 64, 700
    g = ea.AttnGeometry()
    rng = np.random.default_rng(5)
    seq_lens = np.array([200, 33, 600], np.int32)
    sched = ea.Scheduler(nb, 40)
    for i in range(3):
        sched.add_seq(i)
    pre = sched.build_batch([0, 1, 2], seq_lens - 1)
    table = ea.yarn_cos_sin(max_pos)
    kc = np.zeros((nb, 16, hkv, D), np.uint16)
    vc = np.zeros_like(kc)
    kc_d, vc_d = G.cache_dev(kc.copy()), G.cache_dev(vc.copy())
    desc1 = ea.make_desc(g, num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                         max_blocks_per_seq=1, num_blocks=nb)
    # context tokens, then the decode step's own tokens
    for b, seed in ((pre, 31), (sched.build_batch([0, 1, 2], [1, 1, 1]), 32)):
        qkv = synth.normal_bf16((b.num_q_tokens, 10 * hkv * D), seed, synth.TID_Q)
        q_ref = oracle.rope_kv_write(desc1, qkv, b.positions, table, kc, vc, b.slot_mapping)
        q_d = ea.rope_kv_write(g, G.bf16_dev(qkv), G.dev(b.positions), G.dev(table), kc_d, vc_d,
                               G.dev(b.slot_mapping))
    sinks = synth.bf16_bits_to_f32(synth.normal_bf16((64,), 3, synth.TID_SINK)).astype(np.float32)
    desc = ea.make_desc(g, num_seqs=3, num_q_tokens=3, max_q_len=1, max_kv_len=b.max_kv_len,
                        max_blocks_per_seq=40, num_blocks=nb, sum_kv_len=b.sum_kv_len)
    ref, _ = oracle.attn_f64(desc, q_ref, kc, vc, b.block_table, b.seq_lens, None, sinks)
    out = ea.attn_decode(g, q_d, kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens),
                         max_kv_len=b.max_kv_len, sinks=G.dev(sinks), sum_kv_len=b.sum_kv_len)
    torch.cuda.synchronize()
    assert np.array_equal(G.bits_host(q_d), q_ref)
    assert_close(G.bits_host(out), ref, "rope + write + decode")


# ---------------------------------------------------------------- fused with the projection
@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("T,hkv,K,with_bias", [(1, 8, 2880, True), (16, 8, 2880, True),
                                               (17, 8, 256, False), (40, 8, 2880, True),
                                               (64, 8, 2880, True), (64, 1, 128, True),
                                               (33, 2, 640, False)])
def test_projection_rotation_and_write_in_one_launch(G, kv_dtype, T, hkv, K, with_bias):
    """eid_qkv_rope_kv_write against eid_o_proj followed by eid_rope_kv_write on the same
    inputs: q_out and both caches bit for bit (skipped slots and poison included), and the
    two-launch path is itself bit-exact against the oracle's rotation of its projection."""
    nb, max_pos = 24, 3000
    g = ea.AttnGeometry(num_q_heads=8 * hkv, num_kv_heads=hkv, kv_dtype=kv_dtype)
    N = 10 * hkv * D
    rng = np.random.default_rng(T + K)
    hidden = G.bf16_dev(synth.normal_bf16((T, K), 70 + T, synth.TID_Q))
    w_bits = synth.f32_to_bf16_bits((synth.bf16_bits_to_f32(
        synth.normal_bf16((N, K), 71 + T, synth.TID_K)) * (1.5 / np.sqrt(K))).astype(np.float32))
    weight = G.bf16_dev(w_bits)
    bias = G.bf16_dev(synth.normal_bf16((N,), 72 + T, synth.TID_V)) if with_bias else None
    pos = rng.integers(0, max_pos, size=T).astype(np.int32)
    pos[0] = max_pos + 5                                 # clamped into the table
    slots = rng.permutation(nb * 16)[:T].astype(np.int64)
    slots[2::5] = -1
    table = G.dev(ea.yarn_cos_sin(max_pos))
    if kv_dtype == KV_FP8_E4M3:
        fill, dt = 0x5A, np.uint8
        ks = G.dev(np.linspace(0.008, 0.02, hkv).astype(np.float32))
        vs = G.dev(np.linspace(0.02, 0.008, hkv).astype(np.float32))
    else:
        fill, dt, ks, vs = 0xABCD, np.uint16, None, None
    caches = [G.cache_dev(np.full((nb, 16, hkv, D), fill, dt)) for _ in range(4)]
    qkv = ea.o_proj(hidden, weight, bias)
    q_two = ea.rope_kv_write(g, qkv, G.dev(pos), table, caches[0], caches[1], G.dev(slots), ks, vs)
    q_one = ea.qkv_rope_kv_write(g, hidden, weight, bias, G.dev(pos), table, caches[2], caches[3],
                                 G.dev(slots), ks, vs)
    torch.cuda.synchronize()
    assert torch.equal(q_one, q_two)
    assert torch.equal(caches[2], caches[0]) and torch.equal(caches[3], caches[1])
    assert not torch.equal(caches[0], G.cache_dev(np.full((nb, 16, hkv, D), fill, dt)))


def test_fused_projection_argument_errors(G):
    g = ea.AttnGeometry()
    hidden = torch.zeros((65, 128), dtype=torch.bfloat16, device=G.DEV)
    weight = torch.zeros((5120, 128), dtype=torch.bfloat16, device=G.DEV)
    kc = torch.zeros((4, 16, 8, 64), dtype=torch.bfloat16, device=G.DEV)
    pos = torch.zeros(65, dtype=torch.int32, device=G.DEV)
    slots = torch.zeros(65, dtype=torch.int64, device=G.DEV)
    table = G.dev(ea.yarn_cos_sin(16))
    with pytest.raises(ea.EidError) as e:                # more than 64 tokens
        ea.qkv_rope_kv_write(g, hidden, weight, None, pos, table, kc, kc.clone(), slots)
    assert e.value.status == _lib.EID_ERR_UNSUPPORTED
    with pytest.raises(ea.EidError) as e:                # in_features not a multiple of 64
        ea.qkv_rope_kv_write(g, hidden[:4, :96].contiguous(), weight[:, :96].contiguous(), None,
                             pos[:4], table, kc, kc.clone(), slots[:4])
    assert e.value.status == _lib.EID_ERR_INVALID_ARG
    q = ea.qkv_rope_kv_write(g, hidden[:0], weight, None, pos[:0], table, kc, kc.clone(), slots[:0])
    assert q.shape[0] == 0                               # empty batch: nothing launched
