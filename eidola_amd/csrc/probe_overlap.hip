// Measurement probe (not part of the attention ABI): how far do matrix (MFMA) and vector
// (VALU) instructions overlap on a gfx950 SIMD?  Register-only kernels, no memory traffic in
// the timed loop, every SIMD of the device busy.  One iteration = the work of one 16-row tile
// stage of the prefill kernel's inner loop: 18 v_mfma_f32_16x16x32_bf16 (8 score + 10 output)
// and the softmax's vector work on 16 scores per lane (8 max3, 16 exp2, 8 bf16 conversions,
// 4 moves).  Modes:
//   0  MFMA only                      every wave runs the 18 MFMAs
//   1  VALU only                      every wave runs the vector work
//   2  phases                         every wave: 18 MFMAs, then the vector work (what
//                                     compiler-scheduled attention code looks like)
//   3  interleaved                    every wave: one MFMA, then two or three vector
//                                     instructions, a scheduling barrier, and so on
//   4  role split                     8-wave workgroups: waves 0-3 (one per SIMD) run mode 0,
//                                     waves 4-7 run mode 1, side by side on the same SIMDs
//   5  MFMA only, 32x32x16            9 v_mfma_f32_32x32x16_bf16 (the same FLOPs as mode 0)
//   6  interleaved, 32x32x16          9 MFMAs with the same vector work between them
//   7  tile stage, 32x32x16           the prefill kernel's stage with its real dependencies: a
//                                     chain of 4 score MFMAs seeded with 0, 2 row-sum MFMAs
//                                     (16x16x32) and 4 output MFMAs that consume the P made from
//                                     the previous stage's scores, order C0 C1 A0 C2 A1 C3 A2 C4 A3 C5
//   8  mode 7 + the stage's three wave-uniform branches (two on scalars, one on a ballot of the
//      lane maxima)
//   9  mode 8 + the stage's LDS operand reads (4 x 16 bytes and 4 transposing 8-byte reads per
//      lane and stage from a tile that stays put)
// Each launch reports the time per iteration from HIP events and, from inside the kernel, the
// core-clock cycles (s_memtime) and constant-rate ticks (s_memrealtime, 100 MHz) a wave spent
// in its loop: cycles / ticks gives the clock the SIMDs actually ran at under that load, which
// is what turns cycle counts into a fraction of the published (2.4 GHz) peak.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include <utility>

namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float max3(float a, float b, float c) {
  return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  f32x2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
#define SB() __builtin_amdgcn_sched_barrier(0)

struct Vec {  // the vector work's state: 16 scores, a running value that feeds back
  float s[16];
  float m;
  uint32_t p[8];
};

// vector op number `op` of the stage (0..35): 8 max3, then (exp2, exp2, convert) x 8, then 4 moves
template <int OP>
__device__ __forceinline__ void vop(Vec &v, float &mx, f32x4 &z) {
  if constexpr (OP == 0) mx = max3(v.s[0], v.s[1], v.s[2]);
  else if constexpr (OP < 7) mx = max3(mx, v.s[2 * OP + 1], v.s[2 * OP + 2]);
  else if constexpr (OP == 7) mx = __builtin_elementwise_maximum(mx, v.s[15]);
  else if constexpr (OP < 32) {
    constexpr int e = OP - 8, k = e / 3;
    if constexpr (e % 3 != 2) {
      constexpr int i = 2 * k + e % 3;
      // (the argument is kept small and data-dependent so that nothing folds away)
      v.s[i] = __builtin_amdgcn_exp2f(v.s[i] * 0.001f - v.m);  // (stays within [0, 1])
    } else {
      uint32_t w = pack_bf16(v.s[2 * k], v.s[2 * k + 1]);
      asm volatile("" : "+v"(w));
      v.p[k] = w;
    }
  } else {  // four full-rate instructions standing for the accumulator seed's moves
    constexpr int r = OP - 32;
    z[r] = z[r] * 0.5f + mx;
  }
}
constexpr int kVops = 36;
// The exp2 above carries a multiply-subtract (the unfolded softmax: one FMA per score); the
// prefill kernel's folded form has none.  FOLDED drops it.
template <int OP, bool FOLDED>
__device__ __forceinline__ void vop2(Vec &v, float &mx, f32x4 &z) {
  if constexpr (FOLDED && OP >= 8 && OP < 32 && (OP - 8) % 3 != 2) {
    constexpr int i = 2 * ((OP - 8) / 3) + (OP - 8) % 3;
    v.s[i] = __builtin_amdgcn_exp2f(-v.s[i]);  // (settles between 0.5 and 1; the negation is free)
  } else {
    vop<OP>(v, mx, z);
  }
}

template <int... Is, typename F>
__device__ __forceinline__ void sfor_impl(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void sfor(F &&f) {
  sfor_impl(std::make_integer_sequence<int, N>{}, f);
}

// MFMA orders of the tile stage: [0] C0 C1 A0 C2 A1 C3 A2 C4 A3 C5 (modes 7..12),
// [1] A0 C0 A1 C1 A2 C2 A3 C3 C4 C5 (mode 13: scores a third of a stage ahead of their use),
// [2] A0 C0 C1 A1 C2 C3 A2 C4 A3 C5 (mode 14: score steps three apart where possible),
// [3] A0 A1 A2 A3 C0 C1 C2 C3 C4 C5 (mode 15: the chain back to back)
constexpr int kStageOrder[4][10] = {{4, 5, 0, 6, 1, 7, 2, 8, 3, 9},
                                    {0, 4, 1, 5, 2, 6, 3, 7, 8, 9},
                                    {0, 4, 5, 1, 6, 7, 2, 8, 3, 9},
                                    {0, 1, 2, 3, 4, 5, 6, 7, 8, 9}};

template <int MODE>
__global__ __launch_bounds__(512) void overlap_probe_kernel(float *out, unsigned long long *clk,
                                                            int iters, float seed) {
  // More than half of a CU's 160 KB of LDS: at most ONE workgroup is resident per CU, so that a
  // grid of several workgroups per CU loads every SIMD with exactly blockDim / 256 waves.
  // (requested as dynamic LDS at launch; modes 9+ read operands from its first 32 KiB)
  extern __shared__ __align__(16) uint8_t lds_tile[];
  const bool flag_a = iters < 0, flag_b = seed > 1e30f;  // wave-uniform, false, unknown to the compiler
  if (MODE == 9) {
    for (int i = threadIdx.x; i < 8192; i += blockDim.x) ((uint32_t *)lds_tile)[i] = 0x3c003c00u + i;
    __syncthreads();
  }
  const int wave = threadIdx.x >> 6;
  const bool mfma_role = MODE == 0 || MODE == 2 || MODE == 3 || MODE >= 5 ||
                         (MODE == 4 && wave < 4);
  const bool valu_role = MODE == 1 || MODE == 2 || MODE == 3 || MODE >= 6 || (MODE == 4 && wave >= 4);
  bf16x8 a, b;
  for (int i = 0; i < 8; i++) {
    a[i] = (__bf16)(threadIdx.x * 0.001f + i + seed);
    b[i] = (__bf16)(i * 0.5f + seed);
  }
  f32x4 acc[9];
  f32x16 acc32[3];
  for (int i = 0; i < 9; i++) acc[i] = f32x4{0, 0, 0, 0};
  for (int i = 0; i < 3; i++)
    for (int j = 0; j < 16; j++) acc32[i][j] = 0.f;
  Vec v;
  for (int i = 0; i < 16; i++) v.s[i] = threadIdx.x * 0.01f + i + seed;
  for (int i = 0; i < 8; i++) v.p[i] = 0;
  v.m = 0.5f;
  f32x4 z = {0, 0, 0, 0};
  float mx = 0.f;
  const unsigned long long c0 = __builtin_readcyclecounter();  // s_memtime: core clock
  const unsigned long long r0 = wall_clock64();                // s_memrealtime: 100 MHz
  for (int it = 0; it < iters; it++) {
    if constexpr (MODE == 3) {  // one MFMA, then its share of the vector work
      sfor<18>([&](auto s_c) {
        constexpr int s = s_c;
        acc[s % 9] = mfma16(a, b, acc[s % 9]);
        sfor<kVops>([&](auto op) {
          if constexpr (op * 18 / kVops == s) vop2<op, true>(v, mx, z);
        });
        SB();
      });
    } else if constexpr (MODE == 6) {
      sfor<9>([&](auto s_c) {
        constexpr int s = s_c;
        acc32[s % 3] = mfma32(a, b, acc32[s % 3]);
        sfor<kVops>([&](auto op) {
          if constexpr (op * 9 / kVops == s) vop2<op, true>(v, mx, z);
        });
        SB();
      });
    } else if constexpr (MODE >= 7) {
      // (modes 10..12 are mode 7 with one of its three dependencies cut: 10 the score chain (each
      // step seeded with 0), 11 scores -> vector work, 12 P -> output MFMAs)
      constexpr bool kChain = MODE != 10, kS2V = MODE != 11, kP2M = MODE != 12;
      // P of the previous stage's scores feeds C; A makes the next stage's scores
      bf16x8 pa = kP2M ? __builtin_bit_cast(bf16x8, u32x4{v.p[0], v.p[1], v.p[2], v.p[3]}) : a;
      bf16x8 pb = kP2M ? __builtin_bit_cast(bf16x8, u32x4{v.p[4], v.p[5], v.p[6], v.p[7]}) : b;
      f32x16 sx[4];
      f32x16 sn;
      bf16x8 ka[4] = {a, a, a, a}, va[4] = {b, b, b, b};
      if constexpr (MODE == 9) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          ka[j] = *(const bf16x8 *)(lds_tile + (threadIdx.x & 31) * 144 + (threadIdx.x & 32) / 2 + 32 * j);
          typedef short s16x4_t __attribute__((ext_vector_type(4)));
          typedef __attribute__((address_space(3))) s16x4_t lds_s16x4;
          auto t0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lds_tile + 16384 + (threadIdx.x & 15) * 160 + 64 * j));
          auto t1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lds_tile + 16384 + (threadIdx.x & 15) * 160 + 64 * j + 8));
          va[j] = __builtin_bit_cast(bf16x8, u32x4{__builtin_bit_cast(u32x2, t0)[0], __builtin_bit_cast(u32x2, t0)[1],
                                                   __builtin_bit_cast(u32x2, t1)[0], __builtin_bit_cast(u32x2, t1)[1]});
        }
      }
      sfor<10>([&](auto s_c) {
        constexpr int s = s_c;
        // MFMA of slot s: codes 0..3 = score step, 4..5 = row sums, 6..9 = output MFMAs
        constexpr int code = kStageOrder[MODE == 13 ? 1 : MODE == 14 ? 2 : MODE == 15 ? 3 : 0][s];
        if constexpr (code == 4) acc[0] = mfma16(a, pa, acc[0]);
        else if constexpr (code == 5) acc[0] = mfma16(a, pb, acc[0]);
        else if constexpr (code == 0) {
          f32x16 zero;
#pragma unroll
          for (int i = 0; i < 16; i++) zero[i] = 0.f;
          sn = mfma32(ka[0], b, zero);
        } else if constexpr (code < 4) {
          if constexpr (kChain) sn = mfma32(ka[code], b, sn);
          else {
            f32x16 zero;
#pragma unroll
            for (int i = 0; i < 16; i++) zero[i] = 0.f;
            sx[code] = mfma32(ka[code], b, zero);
          }
        } else acc32[code & 1] = mfma32(va[code - 6], (code < 8 ? pa : pb), acc32[code & 1]);
        sfor<kVops - 4>([&](auto op) {
          if constexpr (op * 10 / (kVops - 4) == s) {
            if constexpr ((MODE == 8 || MODE == 9) && op == 0) {
              if (flag_a) v.s[0] -= v.m;   // (never true; wave-uniform scalar conditions)
              if (flag_b) v.s[1] = -v.s[1];
            }
            vop2<op, true>(v, mx, z);
            if constexpr ((MODE == 8 || MODE == 9) && op == 7) {
              if (__builtin_amdgcn_ballot_w64(mx > 60.f) != 0) v.m += 1.0f;  // (never true)
            }
          }
        });
        SB();
      });
      if constexpr (!kChain) {  // (consumed, so that the MFMAs stay)
#pragma unroll
        for (int j = 1; j < 4; j++) acc[1 + j][0] += sx[j][0];
      }
      if constexpr (kS2V) {
#pragma unroll
        for (int i = 0; i < 16; i++) v.s[i] = sn[i] * 1e-30f + v.s[i];  // next stage's scores depend on A
      } else {
        acc[8][0] += sn[0];
      }
    } else if constexpr (MODE == 5) {
#pragma unroll
      for (int i = 0; i < 9; i++) acc32[i % 3] = mfma32(a, b, acc32[i % 3]);
    } else {
      if (mfma_role) {
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
          for (int i = 0; i < 9; i++) acc[i] = mfma16(a, b, acc[i]);
      }
      if (MODE == 2) SB();
      if (valu_role) sfor<kVops>([&](auto op) { vop2<op, true>(v, mx, z); });
    }
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  const unsigned long long r1 = wall_clock64();
  float r = v.m + z[0] + z[1] + z[2] + z[3] + mx;
  for (int i = 0; i < 9; i++) r += acc[i][0] + acc[i][3];
  for (int i = 0; i < 3; i++) r += acc32[i][0] + acc32[i][15];
  for (int i = 0; i < 16; i++) r += v.s[i];
  for (int i = 0; i < 8; i++) r += (float)v.p[i];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
  if ((threadIdx.x & 63) == 0) {  // per wave: cycles and ticks spent in the loop
    const size_t w = (size_t)blockIdx.x * (blockDim.x >> 6) + wave;
    clk[2 * w] = c1 - c0;
    clk[2 * w + 1] = r1 - r0;
  }
}

template <int MODE>
hipError_t launch(float *out, unsigned long long *clk, int wgs, int block, int iters, hipStream_t st) {
  constexpr int kOccupyBytes = 96 * 1024;
  hipError_t e = hipFuncSetAttribute((const void *)overlap_probe_kernel<MODE>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kOccupyBytes);
  if (e != hipSuccess) return e;
  overlap_probe_kernel<MODE><<<wgs, block, kOccupyBytes, st>>>(out, clk, iters, 0.25f);
  return hipGetLastError();
}

}  // namespace

extern "C" {

// Runs one mode of the probe: `num_wgs` workgroups (several per compute unit; one is resident
// per CU at a time) of 4 * `waves_per_simd` (1 or 2) waves, `iters` iterations per wave.
// out: at least num_wgs * 512 floats, clk: at least num_wgs * 8 * 2 u64 (per wave: core cycles,
// 100 MHz ticks), both device memory of the caller's.  Mode 4 always runs 8-wave workgroups
// (two waves per SIMD).  Returns 0, or the hipError_t of the failed launch.
int eid_probe_overlap(int mode, int waves_per_simd, int num_wgs, int iters, float *out,
                      unsigned long long *clk, void *stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int block = (mode == 4 || waves_per_simd == 2) ? 512 : 256;
  switch (mode) {
    case 0: return (int)launch<0>(out, clk, num_wgs, block, iters, st);
    case 1: return (int)launch<1>(out, clk, num_wgs, block, iters, st);
    case 2: return (int)launch<2>(out, clk, num_wgs, block, iters, st);
    case 3: return (int)launch<3>(out, clk, num_wgs, block, iters, st);
    case 4: return (int)launch<4>(out, clk, num_wgs, block, iters, st);
    case 5: return (int)launch<5>(out, clk, num_wgs, block, iters, st);
    case 6: return (int)launch<6>(out, clk, num_wgs, block, iters, st);
    case 7: return (int)launch<7>(out, clk, num_wgs, block, iters, st);
    case 8: return (int)launch<8>(out, clk, num_wgs, block, iters, st);
    case 9: return (int)launch<9>(out, clk, num_wgs, block, iters, st);
    case 10: return (int)launch<10>(out, clk, num_wgs, block, iters, st);
    case 11: return (int)launch<11>(out, clk, num_wgs, block, iters, st);
    case 12: return (int)launch<12>(out, clk, num_wgs, block, iters, st);
    case 13: return (int)launch<13>(out, clk, num_wgs, block, iters, st);
    case 14: return (int)launch<14>(out, clk, num_wgs, block, iters, st);
    case 15: return (int)launch<15>(out, clk, num_wgs, block, iters, st);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // extern "C"
