"""A decode step captured into a HIP graph ONCE and replayed after the device-side sequence
lengths have grown: the graph must serve the new lengths (the newest key included, the fused
KV write at the new position), also when the capturing call was handed host copies of the
lengths and the block table.  Under capture the library ignores those copies: a plan made
from them (exact grid, partition, item list by value) would be frozen into the graph."""
import numpy as np
import pytest
import torch

import eidola_amd as ea
from eidola_amd import KV_BF16, KV_FP8_E4M3, synth

from helpers import (make_batch, logical_tensors, cpu_caches, oracle_out, assert_close,
                     fp8_scales)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


@pytest.mark.parametrize("kv_dtype", [KV_BF16, KV_FP8_E4M3])
@pytest.mark.parametrize("window", [0, 128])
def test_graph_captured_once_serves_growing_sequences(G, kv_dtype, window):
    grow = 3
    start = np.array([700, 33, 2500, 127, 1152, 15])
    full = make_batch(start + grow, [1] * len(start), window=window, kv_dtype=kv_dtype, seed=23)
    g = full.geom
    q, k, v, sinks = logical_tensors(full)
    ks, vs = fp8_scales(k, v) if kv_dtype == KV_FP8_E4M3 else (None, None)
    kc, vc = cpu_caches(full, k, v, ks, vs)          # every token of the final lengths
    ends = np.cumsum(full.seq_lens)                    # logical row offsets of the sequences' ends
    kc_d, vc_d = G.gpu_caches(full, k, v, ks, vs)
    S = len(start)
    seq_lens_d = G.dev(start.astype(np.int32))
    k_new = torch.empty((S, 8, 64), dtype=torch.bfloat16, device=G.DEV)
    v_new = torch.empty_like(k_new)

    def newest_rows(lens):   # logical K/V rows of position lens - 1 of every sequence
        idx = ends - (full.seq_lens - lens) - 1
        return G.bf16_dev(k[idx]), G.bf16_dev(v[idx])

    # upper bounds in the descriptor, host copies of the CAPTURE-TIME lengths in the arguments
    call = ea.prepare("eid_attn_decode", g, G.bf16_dev(q), kc_d, vc_d, G.dev(full.block_table),
                      seq_lens_d, max_kv_len=full.max_kv_len, sinks=G.dev(sinks), k_scale=G.dev(ks),
                      v_scale=G.dev(vs), sum_kv_len=int(full.seq_lens.sum()), k_new=k_new, v_new=v_new,
                      seq_lens_host=start.astype(np.int32), block_table_host=full.block_table)
    kn, vn = newest_rows(start)
    k_new.copy_(kn)
    v_new.copy_(vn)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(stream=side.cuda_stream)               # warm-up outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            call(stream=side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for step in range(grow + 1):
        lens = (start + step).astype(np.int32)
        seq_lens_d.copy_(G.dev(lens))
        kn, vn = newest_rows(lens)
        k_new.copy_(kn)
        v_new.copy_(vn)
        # poison the newest slot: the step has to write it itself (fused KV write)
        flat_k, flat_v = kc_d.view(-1, 8, 64), vc_d.view(-1, 8, 64)
        slots = np.array([full.all_slots(s)[lens[s] - 1] for s in range(S)], dtype=np.int64)
        flat_k[G.dev(slots)] = 0x7F if kv_dtype == KV_FP8_E4M3 else float("nan")
        flat_v[G.dev(slots)] = 0x7F if kv_dtype == KV_FP8_E4M3 else float("nan")
        call.out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        b = synth.Batch("grown", g, lens, full.q_lens, full.block_table, full.num_blocks, full.seed)
        ref, _ = oracle_out(b, q, kc, vc, sinks, ks, vs)
        assert_close(G.bits_host(call.out), ref, f"replay after {step} appended tokens")
        # the step's own write put the newest rows where eid_kv_write would have
        assert np.array_equal(G.cache_host(kc_d), kc) and np.array_equal(G.cache_host(vc_d), vc)
