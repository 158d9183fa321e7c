"""The attention block of a decoder layer composed from the library's entry points, as an
engine would chain them for a decode step: QKV projection (eid_o_proj as a plain linear
layer) -> rotary embedding + split + KV write -> paged sink-attention -> output projection
with residual add; two layers (one windowed, one full), each with its own pages and weights.
Checked against the same chain built from the CPU oracle's functions, eagerly and replayed
from a HIP graph."""
import numpy as np
import pytest
import torch

import oracle
import eidola_amd as ea
from eidola_amd import synth

pytestmark = pytest.mark.gpu

H, NQKV, NB, MB = 192, (64 + 2 * 8) * 64, 160, 48


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


def _f32(bits):
    return synth.bf16_bits_to_f32(bits).astype(np.float64)


def _scaled(shape, seed, tid, scale):
    """bf16 bits of N(0, scale^2) values."""
    x = synth.bf16_bits_to_f32(synth.normal_bf16(shape, seed, tid)) * scale
    return synth.f32_to_bf16_bits(x.astype(np.float32))


def test_two_layers_of_attention_blocks_against_the_oracle_chain(G):
    seq_lens = np.array([700, 45, 300, 1], np.int32)   # lengths after this step's token
    S = len(seq_lens)
    geoms = [ea.AttnGeometry(window=128), ea.AttnGeometry()]
    sched = [ea.Scheduler(NB, MB) for _ in geoms]       # one pool of pages per layer
    table = ea.yarn_cos_sin(int(seq_lens.max()) + 1)
    sinks = synth.bf16_bits_to_f32(synth.normal_bf16((64,), 9, synth.TID_SINK)).astype(np.float32)
    desc1 = ea.make_desc(geoms[1], num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                         max_blocks_per_seq=1, num_blocks=NB)
    layers = []
    for l, (g, sc) in enumerate(zip(geoms, sched)):
        for i in range(S):
            sc.add_seq(i)
        kc = np.zeros((NB, 16, 8, 64), np.uint16)
        vc = np.zeros_like(kc)
        # the context: earlier tokens of every sequence, written by the same fused kernel
        pre_ids = [i for i in range(S) if seq_lens[i] > 1]
        pre = sc.build_batch(pre_ids, [int(seq_lens[i] - 1) for i in pre_ids])
        qkv_pre = synth.normal_bf16((pre.num_q_tokens, NQKV), 40 + l, synth.TID_K)
        kc_d, vc_d = G.cache_dev(kc.copy()), G.cache_dev(vc.copy())
        oracle.rope_kv_write(desc1, qkv_pre, pre.positions, table, kc, vc, pre.slot_mapping)
        ea.rope_kv_write(g, G.bf16_dev(qkv_pre), G.dev(pre.positions), G.dev(table), kc_d, vc_d,
                         G.dev(pre.slot_mapping))
        b = sc.build_batch(list(range(S)), [1] * S)
        assert np.array_equal(b.seq_lens, seq_lens)
        layers.append(dict(
            g=g, b=b, kc=kc, vc=vc, kc_d=kc_d, vc_d=vc_d,
            wqkv=_scaled((NQKV, H), 50 + l, synth.TID_Q, 0.07),
            bqkv=_scaled((NQKV,), 52 + l, synth.TID_Q, 0.1),
            wo=_scaled((H, 4096), 54 + l, synth.TID_V, 0.02),
            bo=_scaled((H,), 56 + l, synth.TID_V, 0.1)))
    hidden0 = _scaled((S, H), 60, synth.TID_Q, 1.0)

    # ---- the oracle's chain, fed with its own intermediates
    hid = hidden0.copy()
    for L in layers:
        b = L["b"]
        qkv, _ = oracle.o_proj(hid, L["wqkv"], L["bqkv"])
        q = oracle.rope_kv_write(desc1, qkv, b.positions, table, L["kc"], L["vc"], b.slot_mapping)
        desc = ea.make_desc(L["g"], num_seqs=S, num_q_tokens=S, max_q_len=1,
                            max_kv_len=b.max_kv_len, max_blocks_per_seq=MB, num_blocks=NB)
        o, _ = oracle.attn_f64(desc, q, L["kc"], L["vc"], b.block_table, b.seq_lens, None, sinks)
        o_bits = synth.f32_to_bf16_bits(o.astype(np.float32))
        hid, _ = oracle.o_proj(o_bits.reshape(S, 4096), L["wo"], L["bo"], hid)
    ref = _f32(hid)

    # ---- the library's chain
    dev = {k: [G.bf16_dev(L[k]) for L in layers] for k in ("wqkv", "bqkv", "wo", "bo")}
    hidden0_d = G.bf16_dev(hidden0)
    hidden = hidden0_d.clone()
    qkv_d = torch.empty((S, NQKV), dtype=torch.bfloat16, device=G.DEV)
    q_d = torch.empty((S, 64, 64), dtype=torch.bfloat16, device=G.DEV)
    pos_d, tab_d, sinks_d = G.dev(layers[0]["b"].positions), G.dev(table), G.dev(sinks)
    calls, slots = [], []
    for L in layers:
        b = L["b"]
        calls.append(ea.prepare("eid_attn_decode", L["g"], q_d, L["kc_d"], L["vc_d"],
                                G.dev(b.block_table), G.dev(b.seq_lens), None,
                                max_kv_len=b.max_kv_len, sinks=sinks_d, sum_kv_len=b.sum_kv_len,
                                seq_lens_host=b.seq_lens))
        slots.append(G.dev(b.slot_mapping))

    def step(stream=None, fused_qkv=False):
        hidden.copy_(hidden0_d)
        for l, L in enumerate(layers):
            if fused_qkv:   # projection, rotation and KV write in one launch: same bits
                ea.qkv_rope_kv_write(L["g"], hidden, dev["wqkv"][l], dev["bqkv"][l], pos_d, tab_d,
                                     L["kc_d"], L["vc_d"], slots[l], q_out=q_d)
            else:
                ea.o_proj(hidden, dev["wqkv"][l], dev["bqkv"][l], out=qkv_d)
                ea.rope_kv_write(L["g"], qkv_d, pos_d, tab_d, L["kc_d"], L["vc_d"], slots[l],
                                 q_out=q_d)
            calls[l](stream=stream)
            ea.o_proj(calls[l].out, dev["wo"][l], dev["bo"][l], residual=hidden, out=hidden)

    step()
    torch.cuda.synchronize()
    eager = hidden.clone()
    got = _f32(G.bits_host(eager))
    err = np.abs(got - ref)
    # every stage rounds to bf16 once; the two chains feed on their own intermediates
    assert err.max() <= 3e-2 and err.mean() <= 3e-3, (err.max(), err.mean())
    # the new tokens' rows are in the caches, bit for bit (identical qkv rounding permitting:
    # compare the pages of the oracle's chain with a one-ulp allowance on K, exactly on count)
    for L in layers:
        kd = _f32(G.cache_host(L["kc_d"]))
        assert np.abs(kd - _f32(L["kc"])).max() <= 0.15
    step(fused_qkv=True)
    torch.cuda.synchronize()
    assert torch.equal(hidden, eager)
    # the same chain from one HIP graph, twice, with eager work in between
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(side.cuda_stream, fused_qkv=True)
        side.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=side):
            step(side.cuda_stream, fused_qkv=True)
    torch.cuda.synchronize()
    for _ in range(2):
        hidden.zero_()
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(hidden, eager)
