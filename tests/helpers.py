"""Shared builders for the parity tests: small seeded batches, CPU caches, comparisons."""
import numpy as np

import oracle
from eidola_amd import KV_BF16, KV_FP8_E4M3, AttnGeometry, make_desc
from eidola_amd import synth

MAX_ABS_TOL = 2e-2   # attention output tolerance (bf16 out, fp32 accumulate) vs fp64 oracle
MEAN_ABS_TOL = 2e-3


def make_batch(seq_lens, q_lens, *, num_blocks=None, seed=11, window=0, kv_dtype=KV_BF16,
               num_kv_heads=8, partition=0, shuffle=True):
    seq_lens = np.asarray(seq_lens)
    q_lens = np.asarray(q_lens)
    need = int(((seq_lens + 15) // 16).sum())
    nb = num_blocks or need + 7
    geom = AttnGeometry(num_q_heads=8 * num_kv_heads, num_kv_heads=num_kv_heads, window=window,
                        kv_dtype=kv_dtype, partition_size=partition)
    if shuffle:
        bt = synth.build_block_table(seq_lens, nb, seed)
    else:
        bt = synth.build_block_table(seq_lens, nb, seed)
        ident = np.arange(nb, dtype=np.int32)
        off = 0
        for s, L in enumerate(seq_lens):
            n = (int(L) + 15) // 16
            bt[s, :n] = ident[off:off + n]
            off += n
    return synth.Batch("test", geom, seq_lens, q_lens, bt, nb, seed)


def desc_of(batch):
    return make_desc(batch.geom, num_seqs=batch.num_seqs, num_q_tokens=batch.num_q_tokens,
                     max_q_len=batch.max_q_len, max_kv_len=batch.max_kv_len,
                     max_blocks_per_seq=batch.block_table.shape[1], num_blocks=batch.num_blocks)


def logical_tensors(batch, seed=None):
    """Q [T,Hq,D], per-sequence logical K/V [sum L, Hkv, D] (bf16 bits), sinks fp32 [Hq]."""
    seed = batch.seed if seed is None else seed
    g = batch.geom
    q = synth.normal_bf16((batch.num_q_tokens, g.num_q_heads, g.head_dim), seed, synth.TID_Q)
    tot = int(batch.seq_lens.sum())
    k = synth.normal_bf16((tot, g.num_kv_heads, g.head_dim), seed, synth.TID_K)
    v = synth.normal_bf16((tot, g.num_kv_heads, g.head_dim), seed, synth.TID_V)
    sinks = synth.bf16_bits_to_f32(synth.normal_bf16((g.num_q_heads,), seed, synth.TID_SINK))
    return q, k, v, sinks.astype(np.float32)


def all_slots(batch):
    return np.concatenate([batch.all_slots(s) for s in range(batch.num_seqs)])


def fp8_scales(k, v):
    kf = synth.bf16_bits_to_f32(k)
    vf = synth.bf16_bits_to_f32(v)
    ks = (np.abs(kf).max(axis=(0, 2)) / np.float32(448.0)).astype(np.float32)
    vs = (np.abs(vf).max(axis=(0, 2)) / np.float32(448.0)).astype(np.float32)
    return ks, vs


def empty_caches(batch, poison=True):
    g = batch.geom
    shape = (batch.num_blocks, g.block_size, g.num_kv_heads, g.head_dim)
    if g.kv_dtype == KV_FP8_E4M3:
        fill = 0x7F if poison else 0       # NaN code: any read of an unwritten slot shows
        return np.full(shape, fill, np.uint8), np.full(shape, fill, np.uint8)
    fill = 0x7FC1 if poison else 0         # a bf16 NaN pattern
    return np.full(shape, fill, np.uint16), np.full(shape, fill, np.uint16)


def cpu_caches(batch, k, v, k_scale=None, v_scale=None):
    """Caches filled by the oracle's kv_write with every context token of every sequence."""
    kc, vc = empty_caches(batch)
    oracle.kv_write(desc_of(batch), k, v, kc, vc, all_slots(batch), k_scale, v_scale)
    return kc, vc


def oracle_out(batch, q, kc, vc, sinks, k_scale=None, v_scale=None):
    return oracle.attn_f64(desc_of(batch), q, kc, vc, batch.block_table, batch.seq_lens,
                           batch.cu_seqlens_q, sinks, k_scale, v_scale)


def assert_close(out_bits, ref64, what=""):
    got = synth.bf16_bits_to_f32(out_bits).astype(np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - ref64)
    assert err.max() <= MAX_ABS_TOL, f"{what}: max-abs {err.max():.4g} > {MAX_ABS_TOL}"
    assert err.mean() <= MEAN_ABS_TOL, f"{what}: mean-abs {err.mean():.4g} > {MEAN_ABS_TOL}"
    return err.max(), err.mean()
