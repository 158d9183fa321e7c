"""End to end on the GPU: a small continuous-batching run in which every array the kernels
take comes from the block allocator / batch builder (include/eidola_sched.h), with prefix
reuse between sequences.  Every step's output is checked against the fp64 oracle run on a
CPU mirror of the caches, and the caches are checked against the sequences' logical K/V."""
import numpy as np
import pytest
import torch

import oracle
import eidola_amd as ea
from eidola_amd import synth

from helpers import assert_close

pytestmark = pytest.mark.gpu

VOCAB, MAXPOS, NB, MB = 40, 160, 48, 10


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


def _tables():
    """K, V and Q rows as functions of (token id, position): equal prefixes have equal KV."""
    k = synth.normal_bf16((VOCAB, MAXPOS, 8, 64), 5, synth.TID_K)
    v = synth.normal_bf16((VOCAB, MAXPOS, 8, 64), 5, synth.TID_V)
    q = synth.normal_bf16((VOCAB, MAXPOS, 64, 64), 5, synth.TID_Q)
    sinks = synth.bf16_bits_to_f32(synth.normal_bf16((64,), 5, synth.TID_SINK)).astype(np.float32)
    return k, v, q, sinks


def test_continuous_batching_with_prefix_reuse(G):
    ktab, vtab, qtab, sinks = _tables()
    geom = ea.AttnGeometry()
    sched = ea.Scheduler(NB, MB, prefix_reuse=True)
    rng = np.random.default_rng(3)
    poison = np.uint16(0x7FC0)  # bf16 NaN: a slot read without having been written shows up
    kc = np.full((NB, 16, 8, 64), poison, np.uint16)
    vc = np.full((NB, 16, 8, 64), poison, np.uint16)
    kc_d, vc_d = G.cache_dev(kc.copy()), G.cache_dev(vc.copy())
    tokens = {}      # seq id -> all token ids so far (prompt + generated)
    todo = {}        # seq id -> prompt tokens still to prefill

    def add(sid, prompt):
        cached = sched.add_seq(sid, prompt)
        tokens[sid] = list(prompt[:cached])
        todo[sid] = list(prompt[cached:])
        return cached

    def step(ids, q_lens):
        new = []
        for sid, ql in zip(ids, q_lens):
            take = todo[sid][:ql] if todo[sid] else [int(rng.integers(VOCAB))]
            assert len(take) == ql
            todo[sid] = todo[sid][ql:]
            new += take
        b = sched.build_batch(ids, q_lens, new)
        tok = np.array(new)
        k_new, v_new, q = ktab[tok, b.positions], vtab[tok, b.positions], qtab[tok, b.positions]
        for sid, ql, n in zip(ids, q_lens, np.split(tok, b.cu_seqlens_q[1:-1])):
            tokens[sid] += [int(x) for x in n]
        desc = ea.make_desc(geom, num_seqs=b.num_seqs, num_q_tokens=b.num_q_tokens,
                            max_q_len=b.max_q_len, max_kv_len=b.max_kv_len, max_blocks_per_seq=MB,
                            num_blocks=NB, sum_kv_len=b.sum_kv_len)
        # CPU mirror and oracle
        oracle.kv_write(desc, k_new, v_new, kc, vc, b.slot_mapping)
        ref, _ = oracle.attn_f64(desc, q, kc, vc, b.block_table, b.seq_lens, b.cu_seqlens_q, sinks)
        # the mirror holds exactly the logical K/V of every sequence in the batch
        for r, sid in enumerate(ids):
            L = b.seq_lens[r]
            got = kc[b.block_table[r, : (L + 15) // 16]].reshape(-1, 8, 64)[:L]
            want = ktab[np.array(tokens[sid]), np.arange(L)]
            assert np.array_equal(got, want), (sid, L)
        # GPU
        ea.kv_write(geom, G.bf16_dev(k_new), G.bf16_dev(v_new), kc_d, vc_d, G.dev(b.slot_mapping))
        args = (geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens))
        if b.max_q_len == 1:
            out = ea.attn_decode(*args, max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                                 sum_kv_len=b.sum_kv_len, seq_lens_host=b.seq_lens)
        else:
            # the builder's host arrays go to the library as they are: it plans with them
            out = ea.attn_varlen(*args, G.dev(b.cu_seqlens_q), max_q_len=b.max_q_len,
                                 max_kv_len=b.max_kv_len, sinks=G.dev(sinks),
                                 sum_kv_len=b.sum_kv_len, seq_lens_host=b.seq_lens,
                                 cu_seqlens_q_host=b.cu_seqlens_q)
        torch.cuda.synchronize()
        assert_close(G.bits_host(out), ref, f"step {ids} {q_lens}")
        return b

    head = rng.integers(VOCAB, size=64)
    assert add(0, np.concatenate([head[:40]])) == 0
    assert add(1, rng.integers(VOCAB, size=23)) == 0
    step([0, 1], [40, 23])                       # two prefill chunks in one varlen batch
    for _ in range(3):
        step([1, 0], [1, 1])                     # decode, order of the batch changes
    # a third sequence shares the first 32 tokens of sequence 0: only 5 rows are computed
    assert add(2, np.concatenate([head[:32], rng.integers(VOCAB, size=5)])) == 32
    b = step([2, 0, 1], [5, 1, 1])               # verify-length rows mixed with decodes
    assert b.block_table[0, :2].tolist() == b.block_table[1, :2].tolist()   # shared blocks
    sched.free_seq(0)                            # the shared blocks stay alive through seq 2
    for _ in range(12):
        step([1, 2], [1, 1])
    # a fourth sequence with the same 64-token head finds the blocks sequence 0 left behind
    assert add(3, np.concatenate([head, rng.integers(VOCAB, size=9)])) == 32
    step([3, 2], [41, 1])
    step([3, 1, 2], [1, 1, 1])
    assert torch.equal(kc_d.view(torch.int16).cpu(), torch.from_numpy(kc.view(np.int16)))
