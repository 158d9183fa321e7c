"""Pins for the oracle of the output projection (orc_o_proj, orc_f64_to_bf16).  The reference
holds no model code, so parity with it is unpinned; what pins the oracle: float64 matrix
multiplication by numpy (a library routine the sum reduces to), brute-force nearest-even
rounding in exact rational arithmetic, a case where rounding through fp32 first would give
the wrong bf16, the identity weight, and linearity in the bias and residual terms."""
from fractions import Fraction

import numpy as np
import pytest

import oracle
from eidola_amd import synth


def _f32(bits):
    return synth.bf16_bits_to_f32(np.asarray(bits, np.uint16))


def _nearest_even_bf16(x):
    """Brute force over the two neighbouring bf16 values, decided in exact arithmetic."""
    fx = Fraction(x)
    sign = 0x8000 if fx < 0 else 0
    ax = abs(fx)
    cands = np.arange(0, 0x7F80, dtype=np.uint16)       # all finite non-negative bf16
    vals = _f32(cands).astype(np.float64)
    i = int(np.searchsorted(vals, float(ax), side="right")) - 1
    best = None
    for j in (i - 1, i, i + 1, i + 2):
        if 0 <= j < len(cands):
            d = abs(Fraction(float(vals[j])) - ax)
            key = (d, int(cands[j]) & 1)               # ties: even mantissa first
            if best is None or key < best[0]:
                best = (key, int(cands[j]))
    return sign | best[1]


def test_rounding_is_nearest_even_in_exact_arithmetic():
    rng = np.random.default_rng(5)
    xs = list(rng.standard_normal(300) * 10.0 ** rng.integers(-6, 6, 300))
    one = 1.0
    xs += [0.0, 1.0, -1.0, one + 2.0 ** -8, one + 3 * 2.0 ** -8, -(one + 2.0 ** -8),     # exact ties
           one + 2.0 ** -8 + 2.0 ** -40, one + 2.0 ** -8 - 2.0 ** -40, 3.0e38, 1e-39, 7e-41]
    lib = oracle.lib()
    for x in xs:
        assert lib.orc_f64_to_bf16(float(x)) == _nearest_even_bf16(float(x)), x
    # agrees with the fp32 rule wherever the input is an fp32 value
    f = rng.standard_normal(2000).astype(np.float32)
    got = np.array([lib.orc_f64_to_bf16(float(v)) for v in f], np.uint16)
    assert np.array_equal(got, synth.f32_to_bf16_bits(f))


def test_no_double_rounding():
    # just above the midpoint of 1 and 1 + 2^-7: fp32 would round it onto the midpoint and
    # nearest-even would then fall back to 1.0
    x = 1.0 + 2.0 ** -8 + 2.0 ** -30
    assert np.float32(x) == np.float32(1.0 + 2.0 ** -8)
    assert oracle.lib().orc_f64_to_bf16(x) == 0x3F81
    assert oracle.lib().orc_f64_to_bf16(-x) == 0xBF81
    assert oracle.lib().orc_f64_to_bf16(float("inf")) == 0x7F80
    assert oracle.lib().orc_f64_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0
    assert oracle.lib().orc_f64_to_bf16(3.4e38) == 0x7F80       # past max + half an ulp


@pytest.mark.parametrize("T,N,K,with_bias,with_res", [(1, 16, 64, False, False), (5, 48, 192, True, False),
                                                      (37, 80, 512, True, True), (64, 2880, 256, False, True)])
def test_matches_numpy_float64_matmul(T, N, K, with_bias, with_res):
    a = synth.normal_bf16((T, K), 3, synth.TID_Q)
    w = synth.normal_bf16((N, K), 3, synth.TID_K)
    b = synth.normal_bf16((N,), 3, synth.TID_V) if with_bias else None
    r = synth.normal_bf16((T, N), 3, synth.TID_SINK) if with_res else None
    out, exact = oracle.o_proj(a, w, b, r)
    ref = _f32(a).astype(np.float64) @ _f32(w).astype(np.float64).T
    if with_bias:
        ref += _f32(b).astype(np.float64)[None, :]
    if with_res:
        ref += _f32(r).astype(np.float64)
    # the same sum in another order: equal up to fp64 summation error
    scale = np.abs(_f32(a)).astype(np.float64) @ np.abs(_f32(w)).astype(np.float64).T + 8.0
    assert np.all(np.abs(exact - ref) <= 1e-13 * scale)
    # and the rounded result is the nearest bf16 of the exact one (spot-checked exhaustively
    # by brute force on a sample, by the half-ulp bound everywhere)
    got = _f32(out).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 1e-30))) - 7)
    assert np.all(np.abs(got - exact) <= 0.5 * ulp * (1 + 1e-9))
    idx = np.random.default_rng(0).integers(0, T * N, 50)
    for i in idx:
        assert int(out.reshape(-1)[i]) == _nearest_even_bf16(float(exact.reshape(-1)[i]))


def test_identity_weight_returns_the_input_bits():
    T, K = 9, 128
    a = synth.normal_bf16((T, K), 8, synth.TID_Q)
    eye = synth.f32_to_bf16_bits(np.eye(K, dtype=np.float32))
    out, exact = oracle.o_proj(a, eye)
    assert np.array_equal(out, a)
    perm = np.random.default_rng(1).permutation(K)
    out, _ = oracle.o_proj(a, eye[perm])           # row n of the weight picks input column perm[n]
    assert np.array_equal(out, a[:, perm])


def test_weight_is_out_features_by_in_features():
    # a transposed operand would fail here: N != K and the result is checked entry by entry
    a = synth.f32_to_bf16_bits(np.array([[1.0, 2.0] + [0.0] * 62], np.float32))      # [1, 64]
    w = np.zeros((16, 64), np.float32)
    w[3, 0], w[3, 1], w[5, 1] = 4.0, 0.5, -8.0
    out, exact = oracle.o_proj(a, synth.f32_to_bf16_bits(w))
    want = np.zeros(16)
    want[3], want[5] = 1 * 4.0 + 2 * 0.5, 2 * -8.0
    assert np.array_equal(exact[0], want)


def test_bias_and_residual_enter_linearly_before_the_rounding():
    T, N, K = 6, 32, 64
    a = synth.normal_bf16((T, K), 2, synth.TID_Q)
    w = synth.normal_bf16((N, K), 2, synth.TID_K)
    b = synth.normal_bf16((N,), 2, synth.TID_V)
    r = synth.normal_bf16((T, N), 2, synth.TID_SINK)
    _, e0 = oracle.o_proj(a, w)
    _, e1 = oracle.o_proj(a, w, b, None)
    _, e2 = oracle.o_proj(a, w, None, r)
    _, e3 = oracle.o_proj(a, w, b, r)
    fb, fr = _f32(b).astype(np.float64), _f32(r).astype(np.float64)
    assert np.allclose(e1, e0 + fb[None, :], rtol=0, atol=1e-12)
    assert np.allclose(e2, e0 + fr, rtol=0, atol=1e-12)
    assert np.allclose(e3, e0 + fb[None, :] + fr, rtol=0, atol=1e-12)
