"""eid_attn_decode_noalloc (split-KV partials in the library's static device array) against
eid_attn_decode (partials in a workspace of the caller's) on the same inputs: the kernels are
the same, so outputs must agree bit for bit, and both stay within the attention tolerance of
the fp64 oracle.  Two calls in a row share the array, the second on a smaller batch: whatever
the first left behind must not matter.  Runs alone in a fresh process and after other tests."""
import ctypes as C

import numpy as np
import pytest
import torch

import eidola_amd as ea
from eidola_amd import KV_BF16, KV_FP8_E4M3, _lib
from eidola_amd._lib import AttnArgs

from helpers import (make_batch, logical_tensors, cpu_caches, oracle_out, assert_close,
                     fp8_scales, desc_of)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


def _both(G, seq_lens, *, kv_dtype=KV_BF16, window=0, seed=5, host=False, partition=0):
    """Runs one batch through both entry points; returns nothing, asserts everything."""
    batch = make_batch(seq_lens, [1] * len(seq_lens), seed=seed, window=window, kv_dtype=kv_dtype,
                       partition=partition)
    g = batch.geom
    q, k, v, sinks = logical_tensors(batch)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc_d, vc_d = G.gpu_caches(batch, k, v, ks, vs)
    kw = dict(max_kv_len=batch.max_kv_len, sinks=G.dev(sinks), k_scale=G.dev(ks), v_scale=G.dev(vs),
              sum_kv_len=int(batch.seq_lens.sum()) if host else 0)
    if host:
        kw.update(seq_lens_host=batch.seq_lens, block_table_host=batch.block_table)
    bt, sl, q_d = G.dev(batch.block_table), G.dev(batch.seq_lens), G.bf16_dev(q)
    assert ea.workspace_bytes(desc_of(batch)) <= ea.STATIC_WORKSPACE_BYTES
    out_a = ea.attn_decode(g, q_d, kc_d, vc_d, bt, sl, **kw)
    out_b = torch.full_like(out_a, float("nan"))
    ea.attn_decode_noalloc(g, q_d, kc_d, vc_d, bt, sl, out=out_b, **kw)
    torch.cuda.synchronize()
    a, b = G.bits_host(out_a), G.bits_host(out_b)
    assert np.array_equal(a, b), "static-workspace and caller-workspace outputs differ"
    kc, vc = cpu_caches(batch, k, v, ks, vs)
    ref, _ = oracle_out(batch, q, kc, vc, sinks, ks, vs)
    assert_close(b, ref, "decode through the static workspace")


def test_two_calls_in_a_row_share_the_static_workspace(G):
    # first call: several partitions per sequence (partials of up to 24 partitions are left in
    # the array); second call: fewer, shorter sequences with a different partition layout
    _both(G, [6000, 37, 4100, 1000, 2500, 513, 3333, 64], partition=256)
    _both(G, [700, 1, 300], partition=64)


def test_run_time_partition_and_host_planning(G):
    _both(G, [3000, 129, 5000, 800, 2047, 16], host=True)
    _both(G, [900, 450], host=True)


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
def test_window_and_fp8(G, kv_dtype):
    _both(G, [4000, 100, 2000, 129], kv_dtype=kv_dtype, window=128)
    _both(G, [1500, 2600], kv_dtype=kv_dtype, partition=512)


def test_oversized_batches_are_rejected_on_the_gpu_box_too(G):
    # 64 partitions x 512 sequences: 512 * 64 * 64 cells of 136 bytes = 285 MB of partials
    d = ea.make_desc(ea.AttnGeometry(partition_size=128), num_seqs=512, num_q_tokens=512,
                     max_q_len=1, max_kv_len=8192, max_blocks_per_seq=512, num_blocks=300000)
    assert ea.workspace_bytes(d) > ea.STATIC_WORKSPACE_BYTES
    a = AttnArgs()
    for f in ("q", "out", "k_cache", "v_cache", "block_table", "seq_lens"):
        setattr(a, f, 0x1000)
    lib = ea.load_library()
    assert lib.eid_attn_decode_noalloc(C.byref(d), C.byref(a), None) == _lib.EID_ERR_WORKSPACE
    assert b"static" in lib.eid_last_error()
