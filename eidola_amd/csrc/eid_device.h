// Device-side helpers shared by the gfx950 kernels: vector types, MFMA wrappers,
// cross-lane reductions over the four 16-lane rows of a wavefront, bf16/fp8 packing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace eid {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// Finite stand-in for "no key seen yet": exp2(x - kNegBig) never produces NaN.
constexpr float kNegBig = -1.0e30f;

union Frag8 {  // 8 bf16 = one MFMA 16x16x32 / 32x32x16 operand
  bf16x8 v;
  u32x4 u;
  uint32_t w[4];
};

__device__ __forceinline__ f32x4 mfma16x32(const Frag8 &a, const Frag8 &b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
}

// IEEE-754-2019 maximum (v_maximum3_f32 on gfx950).  fmaxf() in IEEE mode first quiets both
// operands (v_max x, x), which doubles the length of a max tree; maximum() takes them as
// they are and lets a NaN through, which is what a NaN score has to do anyway.
__device__ __forceinline__ float max2(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float max3(float a, float b, float c) {
  return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}

// max / sum over the four lanes {n, n+16, n+32, n+48} that share MFMA column n.
// v_permlane16_swap / v_permlane32_swap exchange 16-lane rows (gfx950).
__device__ __forceinline__ float rowgroup_max(float x) {
  uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = max2(__uint_as_float(r[0]), __uint_as_float(r[1]));
  u = __float_as_uint(x);
  r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return max2(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float rowgroup_sum(float x) {
  uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  u = __float_as_uint(x);
  r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// two fp32 -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  f32x2 f = {lo, hi};
  bf16x2 b = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, b);
}

// 8 fp8-e4m3fn bytes (two dwords) -> 8 bf16, exact widening, two elements per instruction
// (v_cvt_scalef32_pk_bf16_fp8 with a unit scale; op_sel picks the low or high byte pair).
__device__ __forceinline__ void fp8x8_to_bf16x8(uint32_t d0, uint32_t d1, uint32_t out[4]) {
  out[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, 1.0f, false));
  out[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, 1.0f, true));
  out[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, 1.0f, false));
  out[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, 1.0f, true));
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Software round-to-nearest-even onto the OCP e4m3fn grid, saturating at +-448; NaN -> 0x7F.
__device__ __forceinline__ uint32_t fp8_e4m3_encode(float x) {
  const uint32_t u = __float_as_uint(x);
  const uint32_t sign = (u >> 24) & 0x80u;
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return 0x7Fu;
  if (a >= 0x43E00000u) return sign | 0x7Eu;  // |x| >= 448
  if (a >= (121u << 23)) {                    // normal in e4m3: |x| >= 2^-6
    uint32_t r = a + 0x7FFFFu + ((a >> 20) & 1u);
    r >>= 20;  // exponent and 3 mantissa bits, carry propagated
    return sign | (r - (120u << 3));
  }
  // subnormal: multiples of 2^-9; 8 rounds up into the smallest normal (0x08)
  const float y = __uint_as_float(a) * 512.0f;
  return sign | (uint32_t)__float2int_rn(y);
}


// LDS transpose read (gfx950 ds_read_b64_tr_b16).  Within each 16-lane row, treat the
// 16 lanes x 4 halfwords addressed by the lanes as a flat array F[lane*4 + e]; lane i
// receives F[i], F[16+i], F[32+i], F[48+i].
__device__ __forceinline__ u32x2 lds_read_tr16(const void *lds_ptr) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)lds_ptr);
  return __builtin_bit_cast(u32x2, v);
}

// The same for bytes (gfx950 ds_read_b64_tr_b8): within each 16-lane row the lanes address
// 16 x 8 bytes, F[lane*8 + e]; lane i receives F[i], F[16+i], ..., F[112+i] (byte k of the
// result comes from lane 2k + i/8 of the row, its byte i%8).
__device__ __forceinline__ u32x2 lds_read_tr8(const void *lds_ptr) {
  typedef int s32x2 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(3))) s32x2 lds_s32x2;
  s32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_s32x2 *)lds_ptr);
  return __builtin_bit_cast(u32x2, v);
}

}  // namespace eid
