"""GPU parity of eid_o_proj against the CPU oracle.  The kernels sum in fp32 (matrix-core
accumulation, then eight K shares or one running sum), the oracle exactly; the stated
tolerance is therefore

    |hip - exact| <= half a bf16 ulp of the exact value + 2^-20 * sum_k |a w|

(the second term bounds the fp32 summation error of 4096 terms with a wide margin), and at
least 98 % of the outputs must be the oracle's bf16 bit for bit (the rest sit next to a
rounding boundary).  Covered: all three kernels and every tile count of the streaming one, ragged
token and feature counts, bias / residual present or not, the residual updated in place, a
poison canary around the output, and attention followed by the projection."""
import numpy as np
import pytest
import torch

import oracle
import eidola_amd as ea
from eidola_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_helpers
    assert torch.cuda.is_available()
    ea.load_library()
    return gpu_helpers


def _f32(bits):
    return synth.bf16_bits_to_f32(np.asarray(bits, np.uint16))


def _check(out_bits, ref_bits, exact, a, w, what):
    got = _f32(out_bits).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 1e-30))) - 7)
    mag = np.abs(_f32(a)).astype(np.float64) @ np.abs(_f32(w)).astype(np.float64).T
    bound = 0.5 * ulp + 2.0 ** -20 * (mag + 8.0)
    err = np.abs(got - exact)
    assert np.all(err <= bound), f"{what}: worst excess {np.max(err - bound):.3e}"
    same = np.mean(out_bits == ref_bits)
    assert same >= 0.98, f"{what}: only {same:.4f} of the outputs match bit for bit"


def _run(G, T, N, K, with_bias, with_res, seed=4, inplace=False):
    a = synth.normal_bf16((T, K), seed, synth.TID_Q)
    w = synth.normal_bf16((N, K), seed, synth.TID_K)
    b = synth.normal_bf16((N,), seed, synth.TID_V) if with_bias else None
    r = synth.normal_bf16((T, N), seed, synth.TID_SINK) if with_res else None
    ref, exact = oracle.o_proj(a, w, b, r)
    a_d, w_d = G.bf16_dev(a), G.bf16_dev(w)
    b_d = G.bf16_dev(b) if with_bias else None
    r_d = G.bf16_dev(r) if with_res else None
    if inplace:
        out_d = ea.o_proj(a_d, w_d, b_d, r_d, out=r_d)
        torch.cuda.synchronize()
        out = G.bits_host(out_d)
    else:
        # canary rows before and after the output
        buf = torch.full((T + 2, N), -7.0, dtype=torch.bfloat16, device="cuda")
        ea.o_proj(a_d, w_d, b_d, r_d, out=buf[1:T + 1])
        torch.cuda.synchronize()
        host = G.bits_host(buf)
        assert np.all(host[0] == 0xC0E0) and np.all(host[-1] == 0xC0E0), "wrote outside out"
        out = host[1:T + 1]
    _check(out, ref, exact, a, w, f"T={T} N={N} K={K} bias={with_bias} res={with_res}")


@pytest.mark.parametrize("T", [1, 7, 16, 17, 32, 33, 48, 49, 64])
def test_streaming_kernel_every_tile_count(G, T):
    _run(G, T, 2880, 4096, True, True)


@pytest.mark.parametrize("T,N,K", [(3, 16, 64), (20, 48, 128), (64, 144, 576), (5, 4096, 2880),
                                   (64, 2880, 512), (40, 32, 8192)])
@pytest.mark.parametrize("with_bias,with_res", [(False, False), (True, False), (False, True)])
def test_streaming_kernel_shapes(G, T, N, K, with_bias, with_res):
    _run(G, T, N, K, with_bias, with_res, seed=T + N)


# more 16-feature tiles than CUs: two tiles per workgroup (the QKV projection's shape,
# 2880 -> 5120, for every token-tile count), short and ragged K, and a feature count that
# cannot be paired (257 tiles: one tile per workgroup after all)
@pytest.mark.parametrize("T,N,K", [(1, 5120, 2880), (16, 5120, 2880), (17, 5120, 2880),
                                   (33, 5120, 2880), (49, 5120, 2880), (64, 5120, 2880),
                                   (64, 8192, 128), (30, 4160, 4160), (9, 4112, 576)])
def test_streaming_kernel_wide_outputs(G, T, N, K):
    _run(G, T, N, K, True, T % 2 == 0, seed=T + K)


# the 64 x 64 tile (few workgroups) and the 128 x 128 tile (the last three: 276, 288 and 286
# big tiles), with ragged token counts and feature counts that end inside a tile
@pytest.mark.parametrize("T,N,K", [(65, 2880, 4096), (128, 128, 64), (129, 16, 128), (200, 144, 576),
                                   (257, 2880, 512), (1000, 1040, 1024), (2048, 256, 256),
                                   (1500, 2880, 512), (1025, 4096, 128), (2790, 1648, 192)])
@pytest.mark.parametrize("with_bias,with_res", [(False, False), (True, True)])
def test_tiled_kernel_shapes(G, T, N, K, with_bias, with_res):
    _run(G, T, N, K, with_bias, with_res, seed=T + K)


# the two halves of K side by side in one workgroup, on every tile the host chooses from
# (features x tokens): 64 x 64 (320 tokens), 96 x 64 (512; 640 tokens of 2,000 features ending
# inside a tile), 128 x 64 (640), 96 x 128 (900; 700 tokens of 3,008 features), 128 x 128 (1,300)
@pytest.mark.parametrize("T,N,K", [(320, 2880, 4096), (512, 2880, 4096), (640, 2000, 1024), (640, 2880, 4096),
                                   (900, 2880, 4096), (700, 3008, 512), (1300, 2880, 4096)])
def test_split_k_tiles(G, T, N, K):
    _run(G, T, N, K, True, True, seed=T + N + K)


@pytest.mark.parametrize("T,N,K", [(65, 2880, 4096), (128, 128, 64), (129, 16, 128), (200, 144, 576),
                                   (257, 2880, 512), (1000, 1040, 1024), (513, 208, 192),
                                   (2790, 1648, 192)])
@pytest.mark.parametrize("with_bias,with_res", [(False, False), (True, True)])
@pytest.mark.parametrize("kernel", ["wide", "mid"])
def test_wide_kernel_shapes(G, monkeypatch, kernel, T, N, K, with_bias, with_res):
    # the direct-to-LDS kernels (256 x 192 and 128 x 128 tiles) forced onto shapes they would
    # not be chosen for: ragged token and feature tiles, one and many K steps (odd and even
    # counts), a single workgroup
    monkeypatch.setenv("EID_OPROJ_KERNEL", kernel)
    _run(G, T, N, K, with_bias, with_res, seed=T + K + 1)


def test_wide_and_tiled_kernels_agree(G, monkeypatch):
    a = synth.normal_bf16((700, 1024), 21, synth.TID_Q)
    w = synth.normal_bf16((400, 1024), 21, synth.TID_K)
    a_d, w_d = G.bf16_dev(a), G.bf16_dev(w)
    monkeypatch.setenv("EID_OPROJ_KERNEL", "tiled")
    o_t = G.bits_host(ea.o_proj(a_d, w_d))
    monkeypatch.setenv("EID_OPROJ_KERNEL", "wide")
    o_w = G.bits_host(ea.o_proj(a_d, w_d))
    monkeypatch.setenv("EID_OPROJ_KERNEL", "mid")
    o_m = G.bits_host(ea.o_proj(a_d, w_d))
    torch.cuda.synchronize()
    # the same products summed in the same K order by the same MFMA: bit for bit
    assert np.array_equal(o_w, o_m)
    # the 64 x 64 kernel walks the two halves of K side by side here (77 tiles for 256 CUs) and
    # adds the two sums at the end: equal up to one bf16 step on the few boundary cases
    ft, fw = _f32(o_t).astype(np.float64), _f32(o_w).astype(np.float64)
    assert np.mean(o_t == o_w) >= 0.98
    assert np.all(np.abs(ft - fw) <= 2.0 ** -7 * np.maximum(np.abs(ft), np.abs(fw)) + 1e-3)


@pytest.mark.parametrize("T", [33, 300])
def test_residual_updated_in_place(G, T):
    _run(G, T, 2880, 4096, True, True, inplace=True)


def test_prefill_sized_batch_against_the_oracle(G):
    # the bench workload's shape for a chunked-prefill step (4,216 tokens): the wide kernel
    _run(G, 4216, 2880, 4096, True, True, seed=12)


def test_prefill_sized_batch_in_place(G):
    _run(G, 2600, 2880, 4096, True, True, seed=13, inplace=True)  # (128 x 128 direct-to-LDS tiles)


def test_both_kernels_agree_across_the_switch(G):
    # 64 tokens (streaming) and the same 64 tokens as the head of a 65-token batch (tiled)
    a = synth.normal_bf16((65, 4096), 9, synth.TID_Q)
    w = synth.normal_bf16((2880, 4096), 9, synth.TID_K)
    a_d, w_d = G.bf16_dev(a), G.bf16_dev(w)
    o64 = G.bits_host(ea.o_proj(a_d[:64].contiguous(), w_d))
    o65 = G.bits_host(ea.o_proj(a_d, w_d))
    torch.cuda.synchronize()
    f64, f65 = _f32(o64).astype(np.float64), _f32(o65[:64]).astype(np.float64)
    # different summation orders: equal up to one bf16 step on the few boundary cases
    assert np.mean(o64 == o65[:64]) >= 0.98
    assert np.all(np.abs(f64 - f65) <= 2.0 ** -7 * np.maximum(np.abs(f64), np.abs(f65)) + 1e-3)


def test_attention_output_feeds_the_projection_as_it_stands(G):
    """eid_attn_decode's out [T, Hq, 64] is passed on without any reshuffle; the oracle chain
    (attention, bf16 rounding, projection) is the check."""
    from helpers import make_batch, logical_tensors, cpu_caches, oracle_out
    batch = make_batch([300, 1100, 47, 2048, 513], [1] * 5, seed=31)
    q, k, v, sinks = logical_tensors(batch)
    kc, vc = cpu_caches(batch, k, v)
    ref_attn, _ = oracle_out(batch, q, kc, vc, sinks)                  # float64 [T, Hq, D]
    kc_d, vc_d = G.gpu_caches(batch, k, v)
    out_d = G.run_attn(batch, q, kc_d, vc_d, sinks, return_device=True)
    w = synth.normal_bf16((2880, 4096), 6, synth.TID_K)
    b = synth.normal_bf16((2880,), 6, synth.TID_V)
    y_d = ea.o_proj(out_d, G.bf16_dev(w), G.bf16_dev(b))
    torch.cuda.synchronize()
    # project exactly what the attention kernel produced: isolates the projection and pins
    # the (head, dim) -> k index order
    attn_bits = G.bits_host(out_d).reshape(5, 4096)
    ref, exact = oracle.o_proj(attn_bits, w, b)
    _check(G.bits_host(y_d), ref, exact, attn_bits, w, "attention -> projection")
    # and the whole chain against the oracle's attention: the attention tolerance (mean-abs
    # 2e-3 per element) carried through 4096 unit-variance weights, plus the bf16 rounding
    chain = ref_attn.reshape(5, 4096) @ _f32(w).astype(np.float64).T + _f32(b).astype(np.float64)
    got = _f32(G.bits_host(y_d)).astype(np.float64)
    assert np.mean(np.abs(got - chain)) <= 2e-3 * np.sqrt(4096) + 2.0 ** -8 * np.mean(np.abs(chain))
