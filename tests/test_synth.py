"""Seeded generators and the five benchmark configurations."""
import numpy as np

from eidola_amd import synth, KV_FP8_E4M3


def test_stream_is_deterministic_and_roughly_normal():
    a = synth.normal_bf16((1000, 64), 3, synth.TID_K)
    b = synth.normal_bf16((1000, 64), 3, synth.TID_K)
    assert np.array_equal(a, b)
    assert not np.array_equal(a, synth.normal_bf16((1000, 64), 4, synth.TID_K))
    x = synth.bf16_bits_to_f32(a)
    assert abs(x.mean()) < 0.02 and abs(x.std() - 1) < 0.02
    # first_index makes slices of one stream line up
    c = synth.normal_bf16((10,), 3, synth.TID_K, first_index=64)
    assert np.array_equal(c, a.reshape(-1)[64:74])
    assert synth.mix64(0, 0, 0) == np.uint64(0xE220A8397B1DCDAF)   # SplitMix64 known answer


def test_permutation_and_randint():
    p = synth.permutation(1000, 1, synth.TID_PERM)
    assert sorted(p.tolist()) == list(range(1000))
    r = synth.randint(10000, 1, 8192, 2, synth.TID_LEN)
    assert r.min() >= 1 and r.max() <= 8192 and abs(r.mean() - 4096) < 100


def test_config1():
    b = synth.config1()
    assert b.seq_lens.tolist() == [37, 128, 511, 1000] and b.num_blocks == 128
    used = np.concatenate([b.block_table[s, :(L + 15) // 16] for s, L in enumerate(b.seq_lens)])
    assert len(used) == 106 and len(set(used.tolist())) == 106
    assert not np.array_equal(used, np.sort(used))            # shuffled
    assert b.slot_mapping.tolist() == [int(b.all_slots(s)[-1]) for s in range(4)]


def test_config2_to_5_shapes_and_work():
    b2 = synth.config2()
    assert b2.num_seqs == 64 and b2.block_table.shape == (64, 512) and b2.num_blocks == 300_000
    w = synth.algorithmic_work(b2)
    assert w["bytes"] == int(b2.seq_lens.sum()) * 2048 + 64 * 2 * 8192 + 256 + \
        4 * int(((b2.seq_lens - 1) // 16 + 1).sum())
    assert w["flops"] == 16384 * int(b2.seq_lens.sum())
    ww = synth.algorithmic_work(synth.config2(window=128))
    assert ww["ctx_tokens"] == int(np.minimum(b2.seq_lens, 128).sum())
    b3 = synth.config3()
    assert b3.num_q_tokens == 4216 and b3.cu_seqlens_q[8] == 4096 and b3.cu_seqlens_q[-1] == 4216
    prior = b3.seq_lens[:8] - 512
    assert (prior >= 0).all() and (prior <= 4096).all()
    long = synth.algorithmic_work(b3, rows="long")
    assert long["pairs"] == int((512 * prior + 131328).sum())
    b4 = synth.config4()
    assert b4.geom.kv_dtype == KV_FP8_E4M3 and b4.num_seqs == 256
    assert synth.algorithmic_work(b4)["bytes"] > int(b4.seq_lens.sum()) * 1024
    b5 = synth.config5(layer=1)
    assert b5.geom.window == 128 and b5.num_q_tokens == 640 and b5.geom.partition_size == 512
    assert synth.config5(layer=0).geom.window == 0
    # scaled-down twins keep the structure
    s = synth.config5(scale=1 / 64)
    assert s.num_seqs == 128 and s.max_kv_len <= 1024
