"""eid_attn_decode with k_new / v_new (the newest token's KV write fused into the attention
launch) against the two-launch sequence eid_kv_write + eid_attn_decode on the same inputs:
outputs AND the whole cache pool must be identical bit for bit (the fused path takes the same
values through the same arithmetic; only where the row comes from differs), and the output
stays within the attention tolerance of the fp64 oracle.  The newest token's slot is poisoned
before the fused call, so a kernel that read it from the cache instead of from k_new would
produce NaNs."""
import numpy as np
import pytest
import torch

import oracle
import eidola_amd as ea
from eidola_amd import KV_BF16, KV_FP8_E4M3

from helpers import (make_batch, logical_tensors, cpu_caches, oracle_out, assert_close,
                     fp8_scales, all_slots, empty_caches)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


def _run(G, seq_lens, *, kv_dtype=KV_BF16, window=0, hkv=8, partition=0, seed=3, hint=False,
         host=False):
    batch = make_batch(seq_lens, [1] * len(seq_lens), seed=seed, window=window, kv_dtype=kv_dtype,
                       num_kv_heads=hkv, partition=partition)
    g = batch.geom
    q, k, v, sinks = logical_tensors(batch)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    # newest token of every sequence: last logical row of its K/V, and its slot
    ends = np.cumsum(batch.seq_lens) - 1
    slots = all_slots(batch)
    new_slots = slots[ends]
    old = np.ones(len(slots), bool)
    old[ends] = False
    # device caches with every OLDER token written and the newest slots still poisoned
    kc0, vc0 = empty_caches(batch)
    kc_a, vc_a = G.cache_dev(kc0), G.cache_dev(vc0)
    ea.kv_write(g, G.bf16_dev(k[old]), G.bf16_dev(v[old]), kc_a, vc_a, G.dev(slots[old]),
                G.dev(ks), G.dev(vs))
    kc_b, vc_b = kc_a.clone(), vc_a.clone()
    kn_d, vn_d = G.bf16_dev(k[ends]), G.bf16_dev(v[ends])
    kw = dict(max_kv_len=batch.max_kv_len, sinks=G.dev(sinks), k_scale=G.dev(ks), v_scale=G.dev(vs),
              sum_kv_len=int(batch.seq_lens.sum()) if hint else 0)
    if host:  # the host's item list (and first page ids) instead of the device-side lookup
        kw.update(seq_lens_host=batch.seq_lens, block_table_host=batch.block_table)
    bt, sl, q_d = G.dev(batch.block_table), G.dev(batch.seq_lens), G.bf16_dev(q)
    # A: two launches
    ea.kv_write(g, kn_d, vn_d, kc_a, vc_a, G.dev(new_slots), G.dev(ks), G.dev(vs))
    out_a = ea.attn_decode(g, q_d, kc_a, vc_a, bt, sl, **kw)
    # B: fused
    out_b = ea.attn_decode(g, q_d, kc_b, vc_b, bt, sl, k_new=kn_d, v_new=vn_d, **kw)
    torch.cuda.synchronize()
    a, b = G.bits_host(out_a), G.bits_host(out_b)
    assert np.array_equal(a, b), "fused and two-launch outputs differ"
    assert np.array_equal(G.cache_host(kc_a), G.cache_host(kc_b)), "k_cache differs"
    assert np.array_equal(G.cache_host(vc_a), G.cache_host(vc_b)), "v_cache differs"
    kc, vc = cpu_caches(batch, k, v, ks, vs)
    ref, _ = oracle_out(batch, q, kc, vc, sinks, ks, vs)
    assert_close(b, ref, "fused decode")
    # and the cache equals the oracle's write of every token
    assert np.array_equal(G.cache_host(kc_b), kc) and np.array_equal(G.cache_host(vc_b), vc)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
def test_newest_token_at_every_position_of_a_chunk(G, kv_dtype):
    # lengths around page, chunk and partition boundaries, incl. a sequence that is only its
    # newest token
    _run(G, [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257, 1023, 1024, 1025],
         kv_dtype=kv_dtype)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("partition", [0, 64, 256])
def test_many_partitions(G, kv_dtype, partition):
    _run(G, [4097, 300, 2048, 2049, 1, 777, 6000], kv_dtype=kv_dtype, partition=partition, seed=5)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
def test_sliding_window(G, kv_dtype):
    _run(G, [1, 100, 128, 129, 500, 2048, 4099], kv_dtype=kv_dtype, window=128, seed=6)


@pytest.mark.parametrize("hkv", [1, 2, 4, 16])
def test_other_head_counts(G, hkv):
    _run(G, [33, 700, 64, 1500], hkv=hkv, seed=7)


def test_large_batch_with_launch_hint(G):
    rng = np.random.default_rng(8)
    _run(G, list(rng.integers(1, 3000, size=150)), seed=8, hint=True)
    _run(G, list(rng.integers(1, 400, size=70)), seed=9, kv_dtype=KV_FP8_E4M3)


@pytest.mark.parametrize("hkv,window,partition,hint,host", [
    (8, 0, 0, False, False), (8, 0, 0, True, False), (8, 0, 256, False, False),
    (8, 300, 0, True, False), (16, 0, 0, True, False), (8, 0, 0, True, True), (16, 0, 1024, True, True),
])
def test_fp8_head_pairs_beyond_one_device_fill(G, hkv, window, partition, hint, host):
    """fp8 decode batches too large for the short-span kernel: the split-KV kernel gives every
    wave two KV heads (32 tokens x 2 heads per step).  Newest tokens at every offset of such a
    step, sequence ends inside a step, 8 and 16 KV heads."""
    rng = np.random.default_rng(31)
    lens = list(rng.integers(1500, 2600, size=30)) + list(range(1100, 1134))
    _run(G, lens, kv_dtype=KV_FP8_E4M3, hkv=hkv, window=window, partition=partition, seed=12,
         hint=hint, host=host)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
def test_fused_write_with_the_hosts_item_list(G, kv_dtype):
    """A batch whose items fit the list a launch can carry: the split-KV kernel takes its
    items (and their first page ids) from the kernel arguments and still writes the newest
    tokens on its way."""
    rng = np.random.default_rng(41)
    _run(G, list(rng.integers(1, 8192, size=64)), kv_dtype=kv_dtype, seed=13, hint=True, host=True)


def test_varlen_entry_rejects_the_fused_arguments(G):
    batch = make_batch([40, 50], [2, 1])
    q, k, v, sinks = logical_tensors(batch)
    kc_d, vc_d = G.gpu_caches(batch, k, v)
    kn = torch.zeros((2, 8, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ea.EidError):
        ea.ops._attn_call("eid_attn_varlen", batch.geom, G.bf16_dev(q), kc_d, vc_d,
                          G.dev(batch.block_table), G.dev(batch.seq_lens),
                          G.dev(batch.cu_seqlens_q), 2, batch.max_kv_len, None, None, None, None,
                          None, None, False, 0, kn, kn)
    with pytest.raises(ea.EidError):  # one without the other
        ea.attn_decode(batch.geom, G.bf16_dev(q[:2]), kc_d, vc_d, G.dev(batch.block_table),
                       G.dev(batch.seq_lens), max_kv_len=batch.max_kv_len, k_new=kn)
