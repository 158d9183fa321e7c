// Paged sink-attention kernels for gfx950 (MI355X): one wavefront-level engine shared by
//   * the bandwidth-bound split-KV kernel (decode and short-q verify rows), and
//   * the prefill kernel for long query chunks (K/V tiles shared through LDS),
// plus the cross-partition log-sum-exp merge.
//
// Engine, per wavefront, per chunk of 64 context tokens (four 16-token pages):
//   S^T[token][row] = K[token][:] . Q[row][:]   v_mfma_f32_16x16x32_bf16, tokens on M so a
//        lane's 16 bytes of a K row ARE its A operand: loaded straight from the page (attend),
//        or read from the wave's LDS tile that whole-line loads filled (attend_dma);
//   online softmax in base 2 on the accumulator layout (a lane owns 4 tokens of one row,
//        the row maximum crosses the four 16-lane rows with v_permlane{16,32}_swap);
//   P^T leaves the softmax already in B-operand layout (tokens on the contraction axis);
//   O^T[dim][row] += V^T[dim][token] . P^T[token][row], with V row-major in LDS and read back
//        transposed: bf16 rows by ds_read_b64_tr_b16, the raw bytes of an fp8 cache by
//        ds_read_b64_tr_b8 and widened in registers (attend_dma_pair, attend_dma_fp8).
// "row" = (query token, query head of the KV group): 8 heads share every K/V byte.
#include <atomic>
#include "eid_device.h"
#include "eid_params.h"
#include <hip/hip_ext.h>

#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <type_traits>
#include <utility>

namespace eid {

constexpr float kLazyLog2 = 8.0f;               // slack of the lazily updated softmax maximum
constexpr int kVRowBytes = 144;                 // 128 B of bf16 + 16 B pad (bank spread)
constexpr int kVPageBytes = kBlock * kVRowBytes;  // one 16-token page of V for one KV head
constexpr int kWaveLdsBytes = 4 * kVPageBytes;  // 64 tokens

__device__ __forceinline__ u32x4 ldg128(const uint8_t *p) { return *(const u32x4 *)p; }

// Block tables are read-only for the lifetime of a launch.  Reading them through the
// constant address space keeps wave-uniform page-id loads on the scalar unit whatever else
// the kernel stores, so they never share a wait counter with the K/V vector loads.
typedef const __attribute__((address_space(4))) int32_t *const_i32_ptr;
__device__ __forceinline__ const_i32_ptr as_constant(const int32_t *p) {
  return (const_i32_ptr)(uintptr_t)p;
}

// Row bookkeeping of a wave's NT 16-row tiles.  Row r = 16 nt + (lane % 16) belongs to query
// token tq0 + r / 8, so one per-lane value and four wave-uniform ones describe every tile;
// the bounds are only materialised on chunks that need masking.
struct RowInfo {
  int t_lane;                    // tq0 + (lane % 16) / 8: the row's token in tile 0
  int tq0, qlen, pos0, window;   // wave-uniform
  // absolute position of the row's query token and the first key it may see
  __device__ __forceinline__ void bounds(const int nt, int &pos, int &lo) const {
    const int t = t_lane + 2 * nt;
    pos = pos0 + (t < qlen ? t : tq0);
    lo = window > 0 ? max(0, pos - window + 1) : 0;
  }
};

// Scores, online softmax and PV for one 64-token chunk whose K operands are in registers
// and whose V tile sits in LDS (four 16-token pages of kVRowBytes-padded rows; `v_rd` is
// the lane's transpose-read base).  The V^T operands are fetched once and reused by all NT
// row tiles.
//
// PRE: the Q operands already carry the factor c2 (load_q<NT, true>), so the MFMA result is
// the score in log2 units, and the reference maximum enters as the accumulator's initial
// value: the matrix pipe delivers S * c2 - m and the softmax needs one v_exp_f32 per score,
// no FMA.  A row that has seen no key yet (m == kNegBig) starts from 0 instead.
//
// PAIR (decode rows of an fp8 cache, NT == 1): the wave serves two neighbouring KV heads at
// once.  Its 64 key slots are 32 tokens x 2 heads, slot = 2 * token + head inside each block
// of 16 slots (exactly what a lane group reads from a token row of the cache: full 128-byte
// lines), and its 16 rows are the 16 query heads of the pair, row r belonging to head r / 8.
// A row only attends to the slots of its own head: the others are masked on every chunk.
//
// QLDS (the prefill kernel without lse): the Q operands of row tile nt are read from the wave's
// LDS copy (q_rd, see chunk_pipe) when the tile's turn comes, instead of being held in `qf`.
// V^T operands of a chunk from its LDS tile: [dim tile][page pair].  `v_sw` != 0: rows of 128
// bytes whose 32-byte pairs of segments are permuted by (row / 2) % 4 (tiles written by direct
// global -> LDS loads, see chunk_pipe); dim tile mt then sits at byte (32 mt) ^ v_sw of its row.
template <int VROW>
__device__ __forceinline__ void read_vt(const uint8_t *v_rd, const int v_sw, Frag8 (&vf)[4][2]) {
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      const uint8_t *v_mt = v_rd + ((32 * mt) ^ v_sw);
      const u32x2 a = lds_read_tr16(v_mt + (2 * pr) * (kBlock * VROW));
      const u32x2 b2 = lds_read_tr16(v_mt + (2 * pr + 1) * (kBlock * VROW));
      vf[mt][pr].w[0] = a[0];
      vf[mt][pr].w[1] = a[1];
      vf[mt][pr].w[2] = b2[0];
      vf[mt][pr].w[3] = b2[1];
    }
}

template <int NT, bool PRE, bool PAIR, bool QLDS>
__device__ __forceinline__ void chunk_core(const Frag8 (&kf)[4][2], const Frag8 (&vf)[4][2],
                                           const Frag8 (&qf_regs)[NT][2], const RowInfo &ri,
                                           const int tc, const bool need_mask, const float c2,
                                           float (&m)[NT], f32x4 (&lacc)[NT],
                                           f32x4 (&acc)[NT][4], const uint8_t *q_rd);

template <int NT, int VROW = kVRowBytes, bool PRE = false, bool PAIR = false, bool QLDS = false>
__device__ __forceinline__ void chunk_step(const Frag8 (&kf)[4][2], const uint8_t *v_rd,
                                           const Frag8 (&qf_regs)[NT][2], const RowInfo &ri,
                                           const int tc, const bool need_mask, const float c2,
                                           float (&m)[NT], f32x4 (&lacc)[NT],
                                           f32x4 (&acc)[NT][4], const uint8_t *q_rd = nullptr) {
  Frag8 vf[4][2];
  read_vt<VROW>(v_rd, 0, vf);
  chunk_core<NT, PRE, PAIR, QLDS>(kf, vf, qf_regs, ri, tc, need_mask, c2, m, lacc, acc, q_rd);
}

template <int NT, bool PRE, bool PAIR, bool QLDS>
__device__ __forceinline__ void chunk_core(const Frag8 (&kf)[4][2], const Frag8 (&vf)[4][2],
                                           const Frag8 (&qf_regs)[NT][2], const RowInfo &ri,
                                           const int tc, const bool need_mask, const float c2,
                                           float (&m)[NT], f32x4 (&lacc)[NT],
                                           f32x4 (&acc)[NT][4], const uint8_t *q_rd) {
  const int g = (threadIdx.x & 63) >> 4;
  Frag8 ones;  // bf16 1.0 in every slot: a row of ones in place of V^T yields row sums of P
  ones.u = u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    Frag8 qf_nt[2];
    if constexpr (QLDS) {
      qf_nt[0].u = *(const u32x4 *)(q_rd + (2 * nt) * 1024);
      qf_nt[1].u = *(const u32x4 *)(q_rd + (2 * nt + 1) * 1024);
    } else {
      qf_nt[0] = qf_regs[nt][0];
      qf_nt[1] = qf_regs[nt][1];
    }
    // S^T = K Q^T (raw scores, fp32); the prefill kernel raises its priority around MFMA
    // clusters so that the matrix pipe is fed first when both of a SIMD's waves are ready
    f32x4 S[4];
    const bool fresh = PRE && m[nt] == kNegBig;
    const float base = fresh ? 0.f : m[nt];
    if (NT == 4) __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      f32x4 z = {0.f, 0.f, 0.f, 0.f};
      if (PRE) z = f32x4{-base, -base, -base, -base};
      z = mfma16x32(kf[b][0], qf_nt[0], z);
      S[b] = mfma16x32(kf[b][1], qf_nt[1], z);
    }
    if (NT == 4) __builtin_amdgcn_s_setprio(0);
    if constexpr (PAIR) {
      const bool hi = (threadIdx.x & 8) != 0;  // the row's KV head within the pair
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (((r & 1) != 0) != hi) S[b][r] = -INFINITY;
      if (need_mask) {
        int pos, lo;
        ri.bounds(nt, pos, lo);
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int j = tc + b * (kBlock / 2) + 2 * g + (r >> 1);
            if (j < lo || j > pos) S[b][r] = -INFINITY;
          }
      }
    } else if (need_mask) {
      int pos, lo;
      ri.bounds(nt, pos, lo);
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int j = tc + b * kBlock + 4 * g + r;
          if (j < lo || j > pos) S[b][r] = -INFINITY;
        }
    }
    // row maximum: v_max3 tree over the lane's 16 scores, then across the four lane rows
    float mloc = max3(S[0][0], S[0][1], S[0][2]);
    mloc = max3(mloc, S[0][3], S[1][0]);
    mloc = max3(mloc, S[1][1], S[1][2]);
    mloc = max3(mloc, S[1][3], S[2][0]);
    mloc = max3(mloc, S[2][1], S[2][2]);
    mloc = max3(mloc, S[2][3], S[3][0]);
    mloc = max3(mloc, S[3][1], S[3][2]);
    mloc = max2(mloc, S[3][3]);
    // Lazy rescaling: the reference maximum m only moves when the running maximum has
    // outgrown it by more than kLazyLog2 (in log2 units), so exp2(s - m) stays <= 2^kLazyLog2
    // (exact in the end: numerator and denominator share m) and the accumulators are
    // rescaled on few chunks only.
    if constexpr (PRE) {
      // S holds s - base.  A fresh row moves to its first finite maximum (a fully masked
      // chunk, maximum -inf, leaves it fresh); the others when the excess passes the slack.
      mloc = rowgroup_max(mloc);
      const bool up = mloc > (fresh ? kNegBig : kLazyLog2);
      if (__any(up)) {
        const float shift = up ? mloc : 0.f;
        const float m_new = up ? base + mloc : m[nt];
        const float alpha = fast_exp2(m[nt] - m_new);
        m[nt] = m_new;
#pragma unroll
        for (int r = 0; r < 4; ++r) lacc[nt][r] *= alpha;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[nt][mt][r] *= alpha;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) S[b][r] -= shift;
      }
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) S[b][r] = fast_exp2(S[b][r]);
    } else {
      mloc = rowgroup_max(mloc) * c2;
      if (__any(mloc > m[nt] + kLazyLog2)) {
        const float m_new = mloc > m[nt] + kLazyLog2 ? mloc : m[nt];
        const float alpha = fast_exp2(m[nt] - m_new);
        m[nt] = m_new;
#pragma unroll
        for (int r = 0; r < 4; ++r) lacc[nt][r] *= alpha;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[nt][mt][r] *= alpha;
      }
      const float m_ref = m[nt];
#pragma unroll
      for (int b = 0; b < 4; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) S[b][r] = fast_exp2(__builtin_fmaf(S[b][r], c2, -m_ref));
    }
    // P^T as B operands: pair 0 = pages 0,1; pair 1 = pages 2,3
    Frag8 pf[2];
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      pf[pr].w[0] = pack_bf16(S[2 * pr][0], S[2 * pr][1]);
      pf[pr].w[1] = pack_bf16(S[2 * pr][2], S[2 * pr][3]);
      pf[pr].w[2] = pack_bf16(S[2 * pr + 1][0], S[2 * pr + 1][1]);
      pf[pr].w[3] = pack_bf16(S[2 * pr + 1][2], S[2 * pr + 1][3]);
    }
    // row sums of the bf16-rounded P (the same values the numerator uses), on the MFMA pipe
    if (NT == 4) __builtin_amdgcn_s_setprio(2);
    lacc[nt] = mfma16x32(ones, pf[0], lacc[nt]);
    lacc[nt] = mfma16x32(ones, pf[1], lacc[nt]);
    // O^T += V^T P^T
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) acc[nt][mt] = mfma16x32(vf[mt][pr], pf[pr], acc[nt][mt]);
    if (NT == 4) __builtin_amdgcn_s_setprio(0);
  }
}

// Per-wave time stamps for the measurement aid (AttnParams::timeline).
__device__ __forceinline__ void timeline_start(const AttnParams &p, const int slot) {
  if (!p.timeline) return;
  const unsigned long long t = __builtin_amdgcn_s_memrealtime();
  // HW_ID (register 4, 32 bits) and XCC_ID (register 20, low 4 bits)
  const unsigned hw = __builtin_amdgcn_s_getreg(4 | (31 << 11));
  const unsigned xcc = __builtin_amdgcn_s_getreg(20 | (3 << 11));
  if ((threadIdx.x & 63) == 0) {
    p.timeline[(size_t)slot * 8 + 0] = t;
    p.timeline[(size_t)slot * 8 + 2] = hw;
    p.timeline[(size_t)slot * 8 + 3] = xcc;
  }
}
__device__ __forceinline__ void timeline_mark(const AttnParams &p, const int slot, const int which) {
  if (!p.timeline) return;
  const unsigned long long t = __builtin_amdgcn_s_memrealtime();
  if ((threadIdx.x & 63) == 0) p.timeline[(size_t)slot * 8 + 4 + which] = t;
}
__device__ __forceinline__ void timeline_end(const AttnParams &p, const int slot, const int work) {
  if (!p.timeline) return;
  const unsigned long long t = __builtin_amdgcn_s_memrealtime();
  if ((threadIdx.x & 63) == 0) {
    p.timeline[(size_t)slot * 8 + 1] = t;
    p.timeline[(size_t)slot * 8 + 2] |= (unsigned long long)(unsigned)work << 32;
  }
}

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(<N - 1>).
template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// ---------------------------------------------------------------------------------------
// Software-pipelined chunk of the prefill kernel (PRE = true: softmax factor folded into Q).
//
// A gfx950 SIMD issues matrix and vector instructions through one port: a wave's MFMA takes
// the port for about 9 cycles and then keeps the matrix pipe busy for 16, during which
// vector instructions can issue, but only if they come NEXT in some wave's stream and do not
// depend on that MFMA.  Compiler-scheduled attention code runs the two kinds of work one
// after the other, and a second wave of the SIMD overlaps only partly (the port goes to the
// oldest ready wave).  So the overlap is written into the stream here.  With the four 16-row
// tiles t = 0..3 of the wave:
//   A(t)   8 MFMAs   S(t) = K Q(t)^T - reference (the accumulator's initial value zs[t])
//   B(t)   vector    exp2 of the 16 scores of a lane, conversion to bf16: P(t)
//   R(t)   2 MFMAs   row sums of P(t)
//   PV(t)  8 MFMAs   O(t) += V^T P(t)^T
// the stream is  A(0) | B(0) + A(1),R(0) | B(1) + PV(0),A(2),R(1) | B(2) + PV(1),A(3),R(2) |
// B(3) + PV(2),R(3) | PV(3), where "+" means: one MFMA, then the next few vector
// instructions, a scheduling barrier, and so on, the vector work spread over the stage's
// MFMAs by its issue cost.
//
// The reference of a row is NOT its running maximum.  It is set from the row's first chunks
// (`track`: chunks that need masking, and the wave's first plain chunk, take the lane-local
// maximum as chunk_step does and move the reference when it is outgrown by 2^kLazyLog2) and
// then left alone: exp2(s - reference) may grow far beyond 1 in a later chunk, which costs
// nothing in fp32 / bf16 until it overflows.  The guard against that is the tile's row sum,
// which R(t) delivers before PV(t) is issued: if it is not below 2^60 (this includes inf and
// NaN) the tile's scores are recomputed from the operands still in registers, the reference
// moves to the row's true maximum, O and l are rescaled, and P is rebuilt.  Scores far BELOW
// the reference underflow to 0, which is their correct weight next to a row sum >= 1.
// A plain stage is therefore 16 exp2 + 8 conversions + one compare and one add.
//
// The Q operands come from the wave's own LDS copy (q_rd: fragment (t, half) at
// (2 t + half) * 1024 + lane * 16): all eight fragments plus two tiles of scores would not fit
// 256 VGPRs.
// ---------------------------------------------------------------------------------------
constexpr int kQFragBytes = 64 * 16;  // one Q fragment of a wave in LDS: 16 bytes per lane
constexpr float kRowSumGuard = 1152921504606846976.0f;  // 2^60

template <int I>
using IC = std::integral_constant<int, I>;

// Vector work of a stage, in order: [Q read of tile t + 2] (PRE ops), the tracking block (one
// op, skipped by a wave-uniform branch on most chunks), then (exp2, exp2, convert) x 8.
// Issue cycles: 4; exp2 8.
constexpr int pipe_op_cost(const int op, const int pre) {
  if (op < pre) return 4;
  if (op == pre) return 0;
  const int e = op - (pre + 1);
  return e % 3 != 2 ? 8 : 4;
}
constexpr int pipe_cost_before(const int op, const int pre) {
  int c = 0;
  for (int i = 0; i < op; ++i) c += pipe_op_cost(i, pre);
  return c;
}

// SWZ: the tiles were written by direct global -> LDS loads: 128-byte rows whose 16-byte
// segments are permuted (K: by (row / 2) % 8; V: pairs of segments by (row / 2) % 4).  The
// second half of a lane's K operand is then at `k_rd ^ 16` (passed as k_rd_hi) and V's dim
// tile mt at byte (32 mt) ^ v_sw of its row.
template <int VROW, bool SWZ = false>
__device__ __forceinline__ void chunk_pipe(const uint8_t *k_rd, const uint8_t *k_rd_hi, const int k_tile_stride,
                                           const uint8_t *v_rd, const int v_sw, const uint8_t *q_rd,
                                           bool &maybe_fresh, float (&m)[4], f32x4 (&zs)[4],
                                           float (&l)[4], f32x4 (&acc)[4][4], const RowInfo &ri,
                                           const int tc, const bool need_mask) {
#define EID_SB() __builtin_amdgcn_sched_barrier(0)
  Frag8 ones;
  ones.u = u32x4{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
  asm volatile("" : "+v"(ones.u));  // kept in registers (else rebuilt from constants at every use)
  Frag8 kf[4][2], vf[4][2], qf[2][2];
  f32x4 S[2][4], lt;
  Frag8 P[2][2];
  const bool track = need_mask || maybe_fresh;
  auto read_q = [&](auto t_c) {
    constexpr int t = t_c;
    qf[t & 1][0].u = *(const u32x4 *)(q_rd + (2 * t) * kQFragBytes);
    qf[t & 1][1].u = *(const u32x4 *)(q_rd + (2 * t + 1) * kQFragBytes);
  };
  // ---- operands of the chunk: K first (the first MFMAs wait for them), Q(0), Q(1), V^T ----
#pragma unroll
  for (int b = 0; b < 4; ++b) kf[b][0].u = *(const u32x4 *)(k_rd + b * k_tile_stride);
  read_q(IC<0>{});
#pragma unroll
  for (int b = 0; b < 4; ++b) kf[b][1].u = *(const u32x4 *)(k_rd_hi + b * k_tile_stride);
  read_q(IC<1>{});
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      const uint8_t *v_mt = v_rd + (SWZ ? (32 * mt) ^ v_sw : 32 * mt);
      const u32x2 a = lds_read_tr16(v_mt + (2 * pr) * (kBlock * VROW));
      const u32x2 b2 = lds_read_tr16(v_mt + (2 * pr + 1) * (kBlock * VROW));
      vf[mt][pr].w[0] = a[0];
      vf[mt][pr].w[1] = a[1];
      vf[mt][pr].w[2] = b2[0];
      vf[mt][pr].w[3] = b2[1];
    }
  EID_SB();
  // MFMA j of A(t): first the four token tiles' first halves, then their second halves
  auto mfma_a = [&](auto t_c, auto j_c) {
    constexpr int t = t_c, j = j_c, b = j & 3;
    if constexpr (j < 4) S[t & 1][b] = mfma16x32(kf[b][0], qf[t & 1][0], zs[t]);
    else S[t & 1][b] = mfma16x32(kf[b][1], qf[t & 1][1], S[t & 1][b]);
  };
  // MFMA j of PV(t): the four dim tiles for token pair 0, then for pair 1
  auto mfma_pv = [&](auto t_c, auto j_c) {
    constexpr int t = t_c, j = j_c, pr = j / 4, i = j % 4;
    acc[t][i] = mfma16x32(vf[i][pr], P[t & 1][pr], acc[t][i]);
  };
  // MFMA j of R(t): row sums of P(t) (every lane of a row receives the sum over its 64 keys)
  auto mfma_r = [&](auto t_c, auto j_c) {
    constexpr int t = t_c, j = j_c;
    if constexpr (j == 0) lt = mfma16x32(ones, P[t & 1][0], f32x4{0.f, 0.f, 0.f, 0.f});
    else lt = mfma16x32(ones, P[t & 1][1], lt);
  };
  auto set_ref = [&](auto t_c, const float m_new) {
    constexpr int t = t_c;
    m[t] = m_new;
    const float nb = m_new == kNegBig ? 0.f : -m_new;
    zs[t] = f32x4{nb, nb, nb, nb};
  };
  auto rescale = [&](auto t_c, const float alpha) {
    constexpr int t = t_c;
    l[t] *= alpha;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[t][mt][r] *= alpha;
  };
  auto lane_max = [&](const f32x4 (&Sx)[4]) {
    float mx = max3(Sx[0][0], Sx[0][1], Sx[0][2]);
#pragma unroll
    for (int o = 1; o < 7; ++o)
      mx = max3(mx, Sx[(2 * o + 1) >> 2][(2 * o + 1) & 3], Sx[(2 * o + 2) >> 2][(2 * o + 2) & 3]);
    return max2(mx, Sx[3][3]);
  };
  // The guard of tile t, between R(t) and PV(t); S(t)'s registers and Q(t) are still there.
  auto guard = [&](auto t_c) {
    constexpr int t = t_c;
    if (__any(!(lt[0] < kRowSumGuard))) {  // (rare) some weight of the tile overflowed
      f32x4(&Sx)[4] = S[t & 1];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        Sx[b] = mfma16x32(kf[b][0], qf[t & 1][0], f32x4{0.f, 0.f, 0.f, 0.f});
        Sx[b] = mfma16x32(kf[b][1], qf[t & 1][1], Sx[b]);
      }
      const float mrow = rowgroup_max(lane_max(Sx));  // (plain chunk: every key is visible)
      const bool fresh = m[t] == kNegBig;
      const float m_new = fresh ? mrow : max2(m[t], mrow);
      rescale(t_c, fresh ? 0.f : fast_exp2(m[t] - m_new));
      set_ref(t_c, m_new);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float p0 = fast_exp2(Sx[(2 * k) >> 2][(2 * k) & 3] - m_new);
        const float p1 = fast_exp2(Sx[(2 * k + 1) >> 2][(2 * k + 1) & 3] - m_new);
        P[t & 1][k >> 2].w[k & 3] = pack_bf16(p0, p1);
      }
      lt = mfma16x32(ones, P[t & 1][0], f32x4{0.f, 0.f, 0.f, 0.f});
      lt = mfma16x32(ones, P[t & 1][1], lt);
    }
    l[t] += lt[0];
  };
  __builtin_amdgcn_s_setprio(1);
  static_for<8>([&](auto j) {
    mfma_a(IC<0>{}, j);
    EID_SB();
  });
  // ---- stages ----
  static_for<4>([&](auto nt_c) {
    constexpr int nt = nt_c;
    constexpr bool has_pv = nt > 0, has_a = nt < 3;
    constexpr int NM = (has_pv ? 8 : 0) + (has_a ? 8 : 0) + 2;  // R(nt) sits at NM - 4, NM - 3
    constexpr int NB = NM - 4;                                   // B(nt) is spread over slots 0..NB-1
    constexpr int kPre = (nt == 1 || nt == 2) ? 1 : 0;           // read_q(nt + 1)
    constexpr int NV = kPre + 1 + 24;
    constexpr int total = pipe_cost_before(NV, kPre);
    f32x4(&Sx)[4] = S[nt & 1];
    if constexpr (has_pv) {
      guard(IC<nt - 1>{});  // before PV(nt - 1) and before Q(nt + 1) replaces Q(nt - 1)
      EID_SB();
    }
    auto vop = [&](auto op_c) {
      constexpr int op = op_c, o = op - kPre - 1;
      if constexpr (op < kPre) {
        constexpr int t1 = nt + 1 < 4 ? nt + 1 : 0;  // (never reached for nt == 3)
        read_q(IC<t1>{});
      } else if constexpr (op == kPre) {
        if (track) {  // a masked chunk or the wave's first plain one: the reference follows the maximum
          if (need_mask) {
            int pos, lo;
            ri.bounds(nt, pos, lo);
            const int j0 = tc + 4 * ((threadIdx.x & 63) >> 4);
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int j = j0 + b * kBlock + r;
                if (j < lo || j > pos) Sx[b][r] = -INFINITY;
              }
          }
          const float mloc = lane_max(Sx);
          if (maybe_fresh || __any(mloc > kLazyLog2)) {
            const bool fresh = m[nt] == kNegBig;
            const float base = fresh ? 0.f : m[nt];
            const float mrow = rowgroup_max(mloc);
            const bool up = mrow > (fresh ? kNegBig : kLazyLog2);
            if (__any(up)) {
              const float shift = up ? mrow : 0.f;
              const float m_new = up ? base + mrow : m[nt];
              rescale(nt_c, fast_exp2(m[nt] - m_new));
              set_ref(nt_c, m_new);
#pragma unroll
              for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int r = 0; r < 4; ++r) Sx[b][r] -= shift;
            }
          }
        }
      } else {
        constexpr int e = o, k = e / 3;  // convert k packs exp2 2k and 2k + 1
        if constexpr (e % 3 != 2) {
          constexpr int i = 2 * k + e % 3;
          Sx[i >> 2][i & 3] = fast_exp2(Sx[i >> 2][i & 3]);
        } else {
          uint32_t w = pack_bf16(Sx[(2 * k) >> 2][(2 * k) & 3], Sx[(2 * k + 1) >> 2][(2 * k + 1) & 3]);
          // (pinned here: the optimiser would otherwise sink the exponentials and the conversion
          // to where P is used, behind the next stage's branch)
          asm volatile("" : "+v"(w));
          P[nt & 1][k >> 2].w[k & 3] = w;
        }
      }
    };
    // MFMA in slot s: PV(nt - 1), then A(nt + 1), with R(nt) in slots NM - 4 and NM - 3
    static_for<NM>([&](auto s_c) {
      constexpr int s = s_c;
      if constexpr (s == NM - 4) mfma_r(nt_c, IC<0>{});
      else if constexpr (s == NM - 3) mfma_r(nt_c, IC<1>{});
      else {
        constexpr int q = s < NM - 4 ? s : s - 2;  // index among the stage's other MFMAs
        if constexpr (has_pv && q < 8) mfma_pv(IC<nt - 1>{}, IC<q>{});
        else mfma_a(IC<(nt + 1 < 4 ? nt + 1 : 0)>{}, IC<(has_pv ? q - 8 : q)>{});
      }
      if constexpr (s < NB) {
        static_for<NV>([&](auto op_c) {
          constexpr int op = op_c;
          if constexpr (pipe_cost_before(op, kPre) * NB / total == s) vop(op_c);
        });
      }
      EID_SB();
    });
  });
  guard(IC<3>{});
  EID_SB();
  static_for<8>([&](auto j) {
    mfma_pv(IC<3>{}, j);
    EID_SB();
  });
  __builtin_amdgcn_s_setprio(0);
  if (!need_mask) maybe_fresh = false;  // every row has seen 64 finite scores
#undef EID_SB
}

// 16 bf16 values -> 16 fp8-e4m3fn bytes, RNE of x / scale (the arithmetic of kv_write_kernel)
__device__ __forceinline__ u32x4 quantize16_fp8(const u32x4 lo, const u32x4 hi, const float sc) {
  u32x4 o = {0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const uint32_t wv = j < 8 ? lo[j >> 1] : hi[(j - 8) >> 1];
    const uint32_t h = (wv >> ((j & 1) * 16)) & 0xffffu;
    o[j >> 2] |= fp8_e4m3_encode(__fdiv_rn(bf16_bits_to_f32(h), sc)) << ((j & 3) * 8);
  }
  return o;
}

// One wavefront attends rows [16*NT) over keys [t_begin, t_end) of sequence `s`.
// t_begin is a multiple of 16.  Tokens >= seq_len are never used (K masked, V zeroed).
//
// Fused KV write (decode, NT == 1, p.k_new set): the sequence's newest token, position
// seq_len - 1, has not been written to the cache yet.  The wave whose key range contains it
// takes that row from k_new / v_new instead of from the cache (the lane that would have
// loaded it swaps its registers) and stores it into the cache on the way, in the format
// kv_write_kernel would have used, so the step needs no separate write launch.  Key ranges
// of different partitions are disjoint and every wave owns one KV head: exactly one lane
// group writes each (sequence, head) row, and nobody else reads it in this launch.
// A page id as the kernels use it: clamped into the pool (scalar, one instruction).
__device__ __forceinline__ int clamp_page(const int id, const int last_block) {
  return (int)min((unsigned)id, (unsigned)last_block);
}

// Page ids of a work item's first chunk, when the launch carries them (else have == 0).
struct FirstPages {
  int have = 0;
  int id[4] = {0, 0, 0, 0};
};

// No partials inside the key range (the default `emit` of attend).
struct NoEmit {
  __device__ __forceinline__ int operator()(int) const { return 0; }
};

// Waits until at most `n` of the wave's vector memory operations are outstanding (they
// complete in the order they were issued): the loads issued before the youngest n, stores, say.
__device__ __forceinline__ void wait_vm_all_but(const int n) {
  if (n >= 14) asm volatile("s_waitcnt vmcnt(14)" ::: "memory");
  else if (n >= 11) asm volatile("s_waitcnt vmcnt(11)" ::: "memory");
  else if (n >= 9) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
  else if (n >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (n >= 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if (n >= 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// `emit_every` > 0 (a multiple of the chunk): after every `emit_every` keys from t_begin, except
// at the end of the range, emit(k) is called with k = 0, 1, ...: the caller stores the partial
// of that stretch and resets m / lacc / acc, and the loop goes on with the next stretch, its
// page ids already under way (a range of several partitions walked without a new start).
// emit returns a lower bound on the number of store instructions it issued (attend_dma lets
// that many operations stay outstanding when it next waits for its loads).
template <int NT, bool FP8, bool PAIR = false, class Emit = NoEmit>
__device__ __forceinline__ void attend(const AttnParams &p, const int s, const int kvh,
                                       const int t_begin, const int t_end, const int seq_len,
                                       const int pos_first, const int lo_last,
                                       const Frag8 (&qf)[NT][2], const RowInfo &ri,
                                       uint8_t *wave_lds, float (&m)[NT], f32x4 (&lacc)[NT],
                                       f32x4 (&acc)[NT][4], const FirstPages &first = FirstPages{},
                                       const int emit_every = 0, const Emit emit = Emit{}) {
  const int lane = threadIdx.x & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const int Hkv = p.num_kv_heads;
  constexpr int kElt = FP8 ? 1 : 2;
  const uint32_t row_bytes = (uint32_t)Hkv * kHeadDim * kElt;
  const size_t page_bytes = (size_t)kBlock * row_bytes;
  static_assert(!PAIR || (FP8 && NT == 1), "head pairs: decode rows of an fp8 cache");
  // PAIR: a block of 16 slots is 8 token rows x 2 heads (lane i16 = 2 * token + head), two
  // blocks per page; `kvh` is the first head of the pair.
  const uint32_t lane_off =
      PAIR ? (uint32_t)(i16 >> 1) * row_bytes + (uint32_t)(kvh + (i16 & 1)) * (kHeadDim * kElt) +
                 (uint32_t)g * (16 * kElt)
           : (uint32_t)i16 * row_bytes + (uint32_t)kvh * (kHeadDim * kElt) + (uint32_t)g * (16 * kElt);
  constexpr int kBlkTok = PAIR ? kBlock / 2 : kBlock;  // tokens per block of 16 slots
  const int tok_lane = PAIR ? (i16 >> 1) : i16;        // the lane's token inside its block
  const const_i32_ptr bt = as_constant(p.block_table + (size_t)s * p.max_blocks_per_seq);
  const int nblk_total = (t_end + kBlock - 1) / kBlock;
  // scores enter the softmax as exp2(S * c2 - m): scale, log2(e) and the fp8 K scale in one
  // factor (> 0: softmax_scale is validated, quantisation scales are magnitudes)
  const float c2 = p.softmax_scale * kLog2e * (FP8 ? p.k_scale[PAIR ? kvh + (i16 >> 3) : kvh] : 1.0f);

  uint8_t *lds_wr = wave_lds + i16 * kVRowBytes + g * 32;
  const uint8_t *lds_rd = wave_lds + (4 * g + (i16 >> 2)) * kVRowBytes + 8 * (i16 & 3);

  // Page ids travel through scalar registers: the table row and the index are wave-uniform,
  // so these are scalar loads that never share a wait counter with the K/V vector loads.
  // The ids of iteration i+1 are fetched while iteration i is in flight.
  constexpr int kPages = PAIR ? 2 : 4;
  constexpr int kIter = PAIR ? kChunk / 2 : kChunk;
  constexpr int kBlocks = 4;                 // blocks of 16 slots per iteration
  constexpr int kBpp = kBlocks / kPages;     // blocks per page
  // position of the token this launch writes itself, if it lies in [t_begin, t_end); else -1
  const int pos_new = (NT == 1 && p.k_new && seq_len - 1 >= t_begin && seq_len - 1 < t_end)
                          ? seq_len - 1 : -1;
  int blk[kPages];
  if (first.have) {  // (wave-uniform) the launch brought the first chunk's page ids along
#pragma unroll
    for (int b = 0; b < kPages; ++b) blk[b] = first.id[b];
  } else {
#pragma unroll
    for (int b = 0; b < kPages; ++b) blk[b] = bt[min(t_begin / kBlock + b, nblk_total - 1)];
  }

  int emit_left = emit_every, emit_k = 0;
  for (int ti = t_begin; ti < t_end; ti += kIter) {
    const int nbi = min(kPages, (t_end - ti + kBlock - 1) / kBlock);

    // ---- global loads: each lane takes 32 B (bf16) / 16 B (fp8) of one token row ----
    u32x4 kraw[kBlocks][kElt], vraw[kBlocks][kElt];
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
      for (int e = 0; e < kElt; ++e) {
        kraw[b][e] = u32x4{0, 0, 0, 0};
        vraw[b][e] = u32x4{0, 0, 0, 0};
      }
      if (b / kBpp < nbi) {
        // (clamped here, at its use: at the load it would make the wave wait for the id)
        const size_t page_off = (size_t)clamp_page(blk[b / kBpp], p.last_block) * page_bytes +
                                lane_off + (uint32_t)(b % kBpp) * kBlkTok * row_bytes;
        const uint8_t *kp = p.k_cache + page_off;
        const uint8_t *vp = p.v_cache + page_off;
#pragma unroll
        for (int e = 0; e < kElt; ++e) {
          // (head pairs: a load instruction takes whole 128-byte lines, and nothing of a line
          // is asked for again: the streaming hint is worth a tenth of the run time there)
          kraw[b][e] = PAIR ? __builtin_nontemporal_load((const u32x4 *)(kp + 16 * e)) : ldg128(kp + 16 * e);
          vraw[b][e] = PAIR ? __builtin_nontemporal_load((const u32x4 *)(vp + 16 * e)) : ldg128(vp + 16 * e);
        }
      }
    }
    if (NT == 1 && pos_new >= ti && pos_new < ti + kIter) {  // wave-uniform, once per sequence
      // One 16-byte piece at a time (K then V), so that the rare path adds few live registers
      // to a loop that runs at the register limit of two workgroups per CU.
      const int b_new = (pos_new - ti) / kBlkTok;
      const bool mine = tok_lane == (pos_new & (kBlkTok - 1));
      const size_t src = ((size_t)s * Hkv + (PAIR ? kvh + (i16 & 1) : kvh)) * kHeadDim + g * 16;
      size_t dst = lane_off;
#pragma unroll
      for (int b = 0; b < kBlocks; ++b)
        if (b == b_new)
          dst += (size_t)clamp_page(blk[b / kBpp], p.last_block) * page_bytes +
                 (size_t)(b % kBpp) * kBlkTok * row_bytes;
#pragma unroll
      for (int kv = 0; kv < 2; ++kv) {
        const uint16_t *from = (kv ? p.v_new : p.k_new) + src;
        uint8_t *to = const_cast<uint8_t *>(kv ? p.v_cache : p.k_cache) + dst;
        if constexpr (FP8) {
          const float sc = (kv ? p.v_scale : p.k_scale)[PAIR ? kvh + (i16 & 1) : kvh];
          const u32x4 x = quantize16_fp8(*(const u32x4 *)from, *(const u32x4 *)(from + 8), sc);
          if (mine) {
            *(u32x4 *)to = x;
#pragma unroll
            for (int b = 0; b < kBlocks; ++b)
              if (b == b_new) (kv ? vraw[b][0] : kraw[b][0]) = x;
          }
          asm volatile("" ::: "memory");
        } else {
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const u32x4 x = *(const u32x4 *)(from + 8 * e);
            if (mine) {
              *(u32x4 *)(to + 16 * e) = x;
#pragma unroll
              for (int b = 0; b < kBlocks; ++b)
                if (b == b_new) (kv ? vraw[b][e * (kElt - 1)] : kraw[b][e * (kElt - 1)]) = x;
            }
            asm volatile("" ::: "memory");
          }
        }
      }
    }
    if (ti + kIter < t_end) {
#pragma unroll
      for (int b = 0; b < kPages; ++b) blk[b] = bt[min((ti + kIter) / kBlock + b, nblk_total - 1)];
    }

    {
    const int tc = ti;
    constexpr int sub = 0;

    // ---- V: zero rows past the sequence end, widen fp8, stage in LDS ----
    const bool tail = tc + kIter > seq_len;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      u32x4 v0, v1;
      if constexpr (FP8) {
        uint32_t lo4[4], hi4[4];
        fp8x8_to_bf16x8(vraw[4 * sub + b][0][0], vraw[4 * sub + b][0][1], lo4);
        fp8x8_to_bf16x8(vraw[4 * sub + b][0][2], vraw[4 * sub + b][0][3], hi4);
        v0 = u32x4{lo4[0], lo4[1], lo4[2], lo4[3]};
        v1 = u32x4{hi4[0], hi4[1], hi4[2], hi4[3]};
      } else {
        v0 = vraw[4 * sub + b][0];
        v1 = vraw[4 * sub + b][kElt - 1];
      }
      if (tail) {  // last chunk of the sequence only (kept a real branch, not 8 selects)
        asm volatile("" ::: "memory");
        if (tc + b * kBlkTok + tok_lane >= seq_len) {
          v0 = u32x4{0, 0, 0, 0};
          v1 = u32x4{0, 0, 0, 0};
        }
      }
      *(u32x4 *)(lds_wr + b * kVPageBytes) = v0;
      *(u32x4 *)(lds_wr + b * kVPageBytes + 16) = v1;
    }

    // ---- K operands ----
    Frag8 kf[4][2];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      if constexpr (FP8) {
        fp8x8_to_bf16x8(kraw[4 * sub + b][0][0], kraw[4 * sub + b][0][1], kf[b][0].w);
        fp8x8_to_bf16x8(kraw[4 * sub + b][0][2], kraw[4 * sub + b][0][3], kf[b][1].w);
      } else {
        kf[b][0].u = kraw[4 * sub + b][0];
        kf[b][1].u = kraw[4 * sub + b][kElt - 1];
      }
    }
    const bool need_mask = (tc < lo_last) || (tc + kIter > pos_first + 1);
    chunk_step<NT, kVRowBytes, false, PAIR>(kf, lds_rd, qf, ri, tc, need_mask, c2, m, lacc, acc);
    }  // sub
    if constexpr (!std::is_same<Emit, NoEmit>::value) {
      emit_left -= kIter;
      if (emit_left == 0 && ti + kIter < t_end) {  // (wave-uniform)
        emit(emit_k++);
        emit_left = emit_every;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// The same over a bf16 cache, with the K/V chunk brought in by direct global -> LDS loads.
//
// What the memory system gives a gather of KV pages depends on the shape of a load
// instruction: when 8 consecutive lanes take the eight 16-byte pieces of one 128-byte line
// (a head's row of one token) and the load carries the non-temporal hint, a plain gather of
// the pages runs at 6.6 - 6.9 TB/s; when every line is picked up in halves by two
// instructions and lanes 16 apart, as the MFMA operand layout would have a register load do,
// it runs at 5.8 - 6.2 TB/s, and the hint makes that worse.  A lane cannot both sit in an
// 8-lane line group and hold its own row's operand slice, so the chunk goes through LDS:
// global_load_lds_dwordx4 moves 8 token rows x 128 bytes per instruction into a wave-private
// tile of 64 rows x 128 bytes for K and one for V (segments permuted as in chunk_pipe, which
// keeps the ds_read_b128 K reads and the transposing V reads free of bank conflicts).  The
// operands of a chunk are read into registers first; then the loads of the NEXT chunk are
// issued into the same two tiles, and they are in flight for the whole of this chunk's
// arithmetic: one tile pair per wave is enough, and no staging registers are held.
// Rows past the end of the sequence repeat its last row (finite data, masked scores).
//
// The fused write of the newest token (NT == 1, p.k_new): its row is stored into the cache
// first and the loads of the chunk that holds it are issued after that store has completed,
// so the row arrives with the rest of its page.
// ---------------------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void dma_gptr_t;
typedef __attribute__((address_space(3))) void dma_lptr_t;
constexpr int kDmaTileBytes = kChunk * 128;          // 64 token rows of one KV head
constexpr int kWaveDmaBytes = 2 * kDmaTileBytes;     // K tile, V tile
constexpr int kDmaAux = 2;                           // non-temporal (streaming) loads

template <int NT, class Emit = NoEmit>
__device__ __forceinline__ void attend_dma(const AttnParams &p, const int s, const int kvh,
                                           const int t_begin, const int t_end, const int seq_len,
                                           const int pos_first, const int lo_last,
                                           const Frag8 (&qf)[NT][2], const RowInfo &ri,
                                           uint8_t *wave_lds, float (&m)[NT], f32x4 (&lacc)[NT],
                                           f32x4 (&acc)[NT][4], const FirstPages &first = FirstPages{},
                                           const int emit_every = 0, const Emit emit = Emit{}) {
  const int lane = threadIdx.x & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const uint32_t row_bytes = (uint32_t)p.num_kv_heads * (kHeadDim * 2);
  const size_t page_bytes = (size_t)kBlock * row_bytes;
  const const_i32_ptr bt = as_constant(p.block_table + (size_t)s * p.max_blocks_per_seq);
  const int nblk_total = (t_end + kBlock - 1) / kBlock;
  const float c2 = p.softmax_scale * kLog2e;
  uint8_t *ktile = wave_lds, *vtile = wave_lds + kDmaTileBytes;
  // loader: lane (r, sl) = (lane / 8, lane % 8) fills slot sl of row 8 h + r of a page
  const int dr = lane >> 3, dsl = lane & 7;
  const uint32_t head_off = (uint32_t)kvh * (kHeadDim * 2);
  // operand reads (see chunk_pipe<128, SWZ>)
  const int sw_k = (i16 >> 1) & 7;
  const uint8_t *k_rd = ktile + (uint32_t)i16 * 128 + (uint32_t)((2 * g) ^ sw_k) * 16;
  const uint8_t *k_rd_hi = ktile + (((uint32_t)i16 * 128 + (uint32_t)((2 * g) ^ sw_k) * 16) ^ 16);
  const int v_row = 4 * g + (i16 >> 2);
  const uint8_t *v_rd = vtile + (uint32_t)v_row * 128 + 8 * (i16 & 3);
  const int v_sw = 32 * ((v_row >> 1) & 3);

  auto pages_of = [&](const int ti, int (&blk)[4]) {
#pragma unroll
    for (int b = 0; b < 4; ++b) blk[b] = bt[min(ti / kBlock + b, nblk_total - 1)];
  };
  auto issue = [&](const int ti, const int (&blk)[4]) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const size_t page_off = (size_t)clamp_page(blk[b], p.last_block) * page_bytes + head_off;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int tok = min(ti + b * kBlock + 8 * h + dr, seq_len - 1);
        const size_t off = page_off + (uint32_t)(tok & (kBlock - 1)) * row_bytes;
        const int kseg = dsl ^ (4 * h + (dr >> 1));
        const int vseg = dsl ^ ((dr >> 1) << 1);
        __builtin_amdgcn_global_load_lds((dma_gptr_t *)(p.k_cache + off + kseg * 16),
                                         (dma_lptr_t *)(ktile + (2 * b + h) * 1024), 16, 0, kDmaAux);
        __builtin_amdgcn_global_load_lds((dma_gptr_t *)(p.v_cache + off + vseg * 16),
                                         (dma_lptr_t *)(vtile + (2 * b + h) * 1024), 16, 0, kDmaAux);
      }
    }
  };

  // newest token: into the cache before anything of its page is requested
  if (NT == 1 && p.k_new && seq_len - 1 >= t_begin && seq_len - 1 < t_end) {  // wave-uniform
    const int pos_new = seq_len - 1;
    const int page = clamp_page(bt[pos_new / kBlock], p.last_block);
    if (lane < 16) {
      const int kv = lane >> 3, c = lane & 7;
      const uint16_t *from = (kv ? p.v_new : p.k_new) + ((size_t)s * p.num_kv_heads + kvh) * kHeadDim + c * 8;
      uint8_t *to = const_cast<uint8_t *>(kv ? p.v_cache : p.k_cache) + (size_t)page * page_bytes +
                    (uint32_t)(pos_new & (kBlock - 1)) * row_bytes + head_off + c * 16;
      *(u32x4 *)to = *(const u32x4 *)from;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the row is in place before its page is read
  }

  int blk[4], blk_next[4];
  if (first.have) {
#pragma unroll
    for (int b = 0; b < 4; ++b) blk[b] = first.id[b];
  } else {
    pages_of(t_begin, blk);
  }
  issue(t_begin, blk);
  if (t_begin + kChunk < t_end) pages_of(t_begin + kChunk, blk_next);

  int emit_left = emit_every, emit_k = 0;
  int stores_behind = 0;  // store instructions issued after the loads that are waited for next
  for (int ti = t_begin; ti < t_end; ti += kChunk) {
    // this chunk's tiles have landed (a partial stored since they were requested may still be
    // on its way: stores behind the loads need not be waited for)
    wait_vm_all_but(stores_behind);
    stores_behind = 0;
    Frag8 kf[4][2], vf[4][2];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      kf[b][0].u = *(const u32x4 *)(k_rd + b * (kBlock * 128));
      kf[b][1].u = *(const u32x4 *)(k_rd_hi + b * (kBlock * 128));
    }
    read_vt<128>(v_rd, v_sw, vf);
    // ... and are in registers: the tiles are free for the next chunk, which streams in while
    // this one is computed
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (ti + kChunk < t_end) {
      issue(ti + kChunk, blk_next);
      if (ti + 2 * kChunk < t_end) pages_of(ti + 2 * kChunk, blk_next);
    }
    const bool need_mask = (ti < lo_last) || (ti + kChunk > pos_first + 1);
    chunk_core<NT, false, false, false>(kf, vf, qf, ri, ti, need_mask, c2, m, lacc, acc, nullptr);
    if constexpr (!std::is_same<Emit, NoEmit>::value) {
      emit_left -= kChunk;
      if (emit_left == 0 && ti + kChunk < t_end) {  // (wave-uniform)
        stores_behind = emit(emit_k++);
        emit_left = emit_every;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Head pairs over an fp8 cache (decode rows), the iteration's raw bytes brought in by direct
// global -> LDS loads.  The register path's loads already cover whole 128-byte lines (two
// neighbouring heads' 64-byte rows), so nothing is reshaped: a lane's 16 bytes land at
// block + 16 lane, exactly the register image the K conversion expects, and come back with one
// ds_read_b128.  The V^T operands are read from the raw bytes as well: ds_read_b64_tr_b8
// hands lane i of a 16-lane row byte i of eight 16-byte runs, i.e. one dimension of eight
// key slots, which widened to bf16 is the MFMA operand; no bf16 copy of V is staged in LDS.
// What the detour buys is the same as in attend_dma: once an iteration's raw bytes are in
// registers the NEXT iteration's loads are issued into the same 8 KiB (K and V of 32 tokens
// x 2 heads) and are in flight while this one is converted and multiplied, where the
// register path has nothing in flight during its arithmetic.
// ---------------------------------------------------------------------------------------
constexpr int kPairRawBytes = 4 * 1024;  // one tensor, one iteration
// V blocks sit 128 bytes apart in bank terms: the two blocks that a transposing read touches
// fall into different halves of the banks (1,024 apart: 256.4 us on config 4 against 255.1)
constexpr int kPairVBlock = 1024 + 128;
constexpr int kPairTileBytes = kPairRawBytes + 4 * kPairVBlock;  // raw K, raw V of one iteration
constexpr int kWavePairDmaBytes = 2 * kPairTileBytes;            // two iterations under way

template <class Emit = NoEmit>
__device__ __forceinline__ void attend_dma_pair(const AttnParams &p, const int s, const int kvh,
                                                const int t_begin, const int t_end, const int seq_len,
                                                const int pos_first, const int lo_last,
                                                const Frag8 (&qf)[1][2], const RowInfo &ri,
                                                uint8_t *wave_lds, float (&m)[1], f32x4 (&lacc)[1],
                                                f32x4 (&acc)[1][4], const int emit_every = 0,
                                                const Emit emit = Emit{}) {
  const int lane = threadIdx.x & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const int Hkv = p.num_kv_heads;
  const uint32_t row_bytes = (uint32_t)Hkv * kHeadDim;
  const size_t page_bytes = (size_t)kBlock * row_bytes;
  // a block of 16 slots is 8 token rows x 2 heads (lane i16 = 2 * token + head), two per page
  const uint32_t lane_off = (uint32_t)(i16 >> 1) * row_bytes + (uint32_t)(kvh + (i16 & 1)) * kHeadDim +
                            (uint32_t)g * 16;
  constexpr int kBlkTok = kBlock / 2, kIter = kChunk / 2;
  const int tok_lane = i16 >> 1;
  const const_i32_ptr bt = as_constant(p.block_table + (size_t)s * p.max_blocks_per_seq);
  const int nblk_total = (t_end + kBlock - 1) / kBlock;
  const float c2 = p.softmax_scale * kLog2e * p.k_scale[kvh + (i16 >> 3)];
  // V^T of (dim tile mt, block pair pr): MFMA k index e of lane row g is slot 4 g + e % 4 of block
  // 2 pr + e / 4 (the order P is packed in); lanes 2 e, 2 e + 1 of the row address that slot's 16
  // bytes of dims 16 mt ... 16 mt + 15, which sit at block + 16 (16 mt + slot)
  const uint8_t *k_rd = wave_lds + lane * 16;
  const uint8_t *vt_rd = wave_lds + kPairRawBytes + (i16 >> 3) * kPairVBlock + 64 * g + 8 * (i16 & 7);

  auto pages_of = [&](const int ti, int (&blk)[2]) {
#pragma unroll
    for (int b = 0; b < 2; ++b) blk[b] = bt[min(ti / kBlock + b, nblk_total - 1)];
  };
  // (every block is loaded: past the end of the range the last page comes in again, real and
  // finite data whose scores are masked and whose V rows are zeroed below)
  auto issue = [&](const int tile_off, const int (&blk)[2]) {
    uint8_t *rawk = wave_lds + tile_off, *rawv = rawk + kPairRawBytes;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const size_t off = (size_t)clamp_page(blk[b >> 1], p.last_block) * page_bytes + lane_off +
                         (uint32_t)(b & 1) * kBlkTok * row_bytes;
      __builtin_amdgcn_global_load_lds((dma_gptr_t *)(p.k_cache + off), (dma_lptr_t *)(rawk + b * 1024), 16, 0, kDmaAux);
      __builtin_amdgcn_global_load_lds((dma_gptr_t *)(p.v_cache + off), (dma_lptr_t *)(rawv + b * kPairVBlock), 16, 0, kDmaAux);
    }
  };

  // newest token: quantised and stored into the cache before anything of its page is requested
  if (p.k_new && seq_len - 1 >= t_begin && seq_len - 1 < t_end) {  // wave-uniform
    const int pos_new = seq_len - 1;
    const int page = clamp_page(bt[pos_new / kBlock], p.last_block);
    const bool mine = tok_lane == (pos_new & (kBlkTok - 1));
    const size_t src = ((size_t)s * Hkv + kvh + (i16 & 1)) * kHeadDim + g * 16;
    const size_t dst = (size_t)page * page_bytes + lane_off + (uint32_t)((pos_new & (kBlock - 1)) >= kBlkTok) * kBlkTok * row_bytes;
#pragma unroll
    for (int kv = 0; kv < 2; ++kv) {
      const uint16_t *from = (kv ? p.v_new : p.k_new) + src;
      const float sc = (kv ? p.v_scale : p.k_scale)[kvh + (i16 & 1)];
      const u32x4 x = quantize16_fp8(*(const u32x4 *)from, *(const u32x4 *)(from + 8), sc);
      if (mine) *(u32x4 *)(const_cast<uint8_t *>(kv ? p.v_cache : p.k_cache) + dst) = x;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the row is in place before its page is read
  }

  // two iterations' loads are under way at any time: tile i + 2 is requested into the tile that
  // iteration i has just read into registers
  int blk[2];
  pages_of(t_begin, blk);
  issue(0, blk);
  if (t_begin + kIter < t_end) {
    pages_of(t_begin + kIter, blk);
    issue(kPairTileBytes, blk);
  }
  if (t_begin + 2 * kIter < t_end) pages_of(t_begin + 2 * kIter, blk);

  int emit_left = emit_every, emit_k = 0;
  int stores_last = 0, stores_before = 0;  // store instructions issued after the last / the last but one request
  int tile_off = 0;
  for (int ti = t_begin; ti < t_end; ti += kIter) {
    // this iteration's tile has landed; the next tile's eight loads (and partials stored since this
    // tile was requested) may still be on their way
    wait_vm_all_but(stores_before + (ti + kIter < t_end ? 8 : 0) + stores_last);
    u32x4 kraw[4];
    u32x2 vt[4][2];
#pragma unroll
    for (int b = 0; b < 4; ++b) kraw[b] = *(const u32x4 *)(k_rd + tile_off + b * 1024);
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) vt[mt][pr] = lds_read_tr8(vt_rd + tile_off + pr * (2 * kPairVBlock) + mt * 256);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (ti + 2 * kIter < t_end) {
      issue(tile_off, blk);
      if (ti + 3 * kIter < t_end) pages_of(ti + 3 * kIter, blk);
    }
    tile_off = kPairTileBytes - tile_off;
    // ---- V: zero the slots past the sequence end (whatever the page holds there), widen ----
    if (ti + kIter > seq_len) {  // last iteration of the sequence only
#pragma unroll
      for (int pr = 0; pr < 2; ++pr)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int t = ti + (2 * pr + h) * kBlkTok + 2 * g;  // bytes 0, 1: token t; 2, 3: t + 1
          const uint32_t keep = (t < seq_len ? 0x0000FFFFu : 0u) | (t + 1 < seq_len ? 0xFFFF0000u : 0u);
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) vt[mt][pr][h] &= keep;
        }
    }
    Frag8 kf[4][2], vf[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) fp8x8_to_bf16x8(vt[mt][pr][0], vt[mt][pr][1], vf[mt][pr].w);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      fp8x8_to_bf16x8(kraw[b][0], kraw[b][1], kf[b][0].w);
      fp8x8_to_bf16x8(kraw[b][2], kraw[b][3], kf[b][1].w);
    }
    const bool need_mask = (ti < lo_last) || (ti + kIter > pos_first + 1);
    chunk_core<1, false, true, false>(kf, vf, qf, ri, ti, need_mask, c2, m, lacc, acc, nullptr);
    stores_before = stores_last;
    stores_last = 0;
    if constexpr (!std::is_same<Emit, NoEmit>::value) {
      emit_left -= kIter;
      if (emit_left == 0 && ti + kIter < t_end) {  // (wave-uniform)
        stores_last = emit(emit_k++);
        emit_left = emit_every;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// One KV head per wave over an fp8 cache (rows of several query tokens per sequence: verify
// steps), the chunk's raw bytes brought in by direct global -> LDS loads and two chunks' loads
// under way per wave, as in attend_dma_pair.  A head's row of a token is 64 bytes, half a
// line: a load instruction takes the rows of a whole page (four lanes per row), and a chunk is
// 4 KiB of K and 4 KiB of V in a wave-private tile of 64 rows x 64 bytes each.  Slot (r, pos)
// of a 16-row block holds the row's 16-byte segment pos ^ (r / 4) ^ (2 for odd blocks): the K
// operand reads (ds_read_b128, one row per lane) and the transposing V reads (ds_read_b64_tr_b8,
// rows 4 g ... 4 g + 3 of two neighbouring blocks per lane row) then touch every bank once.
// Rows past the end of the sequence repeat its last row (finite data, masked scores).
// ---------------------------------------------------------------------------------------
constexpr int kFp8TensorBytes = kChunk * kHeadDim;       // 64 rows x 64 bytes
constexpr int kFp8TileBytes = 2 * kFp8TensorBytes;       // K, V of one chunk
constexpr int kWaveFp8DmaBytes = 2 * kFp8TileBytes;      // two chunks under way

template <int NT, class Emit = NoEmit>
__device__ __forceinline__ void attend_dma_fp8(const AttnParams &p, const int s, const int kvh,
                                               const int t_begin, const int t_end, const int seq_len,
                                               const int pos_first, const int lo_last,
                                               const Frag8 (&qf)[NT][2], const RowInfo &ri,
                                               uint8_t *wave_lds, float (&m)[NT], f32x4 (&lacc)[NT],
                                               f32x4 (&acc)[NT][4], const int emit_every = 0,
                                               const Emit emit = Emit{}) {
  const int lane = threadIdx.x & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const uint32_t row_bytes = (uint32_t)p.num_kv_heads * kHeadDim;
  const size_t page_bytes = (size_t)kBlock * row_bytes;
  const const_i32_ptr bt = as_constant(p.block_table + (size_t)s * p.max_blocks_per_seq);
  const int nblk_total = (t_end + kBlock - 1) / kBlock;
  const float c2 = p.softmax_scale * kLog2e * p.k_scale[kvh];
  // loader: lane (r, pos) = (lane / 4, lane % 4) fills slot pos of row r of a block
  const int dr = lane >> 2;
  const uint32_t seg_even = (uint32_t)kvh * kHeadDim + (uint32_t)(((lane & 3) ^ (dr >> 2)) * 16);
  const uint32_t seg_odd = seg_even ^ 32u;
  // K operand of block b: the lane's row i16, segment g (dims 16 g ... 16 g + 15)
  const uint32_t k_rd = (uint32_t)i16 * kHeadDim + (uint32_t)((g ^ (i16 >> 2)) * 16);
  // V^T of (dim tile mt, block pair pr): MFMA k index e of lane row g is row 4 g + e % 4 of block
  // 2 pr + e / 4; lanes 2 e, 2 e + 1 of the lane row address that row's segment mt
  const uint32_t vt_rd = (uint32_t)kFp8TensorBytes + (uint32_t)(i16 >> 3) * 1024 +
                         (uint32_t)(4 * g + ((i16 >> 1) & 3)) * kHeadDim +
                         (uint32_t)((g ^ (2 * (i16 >> 3))) * 16) + 8 * (i16 & 1);

  auto pages_of = [&](const int ti, int (&blk)[4]) {
#pragma unroll
    for (int b = 0; b < 4; ++b) blk[b] = bt[min(ti / kBlock + b, nblk_total - 1)];
  };
  auto issue = [&](const int tile_off, const int ti, const int (&blk)[4]) {
    uint8_t *ktile = wave_lds + tile_off, *vtile = ktile + kFp8TensorBytes;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int tok = min(ti + b * kBlock + dr, seq_len - 1);
      const size_t off = (size_t)clamp_page(blk[b], p.last_block) * page_bytes +
                         (uint32_t)(tok & (kBlock - 1)) * row_bytes + ((b & 1) ? seg_odd : seg_even);
      __builtin_amdgcn_global_load_lds((dma_gptr_t *)(p.k_cache + off), (dma_lptr_t *)(ktile + b * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((dma_gptr_t *)(p.v_cache + off), (dma_lptr_t *)(vtile + b * 1024), 16, 0, 0);
    }
  };

  int blk[4];
  pages_of(t_begin, blk);
  issue(0, t_begin, blk);
  if (t_begin + kChunk < t_end) {
    pages_of(t_begin + kChunk, blk);
    issue(kFp8TileBytes, t_begin + kChunk, blk);
  }
  if (t_begin + 2 * kChunk < t_end) pages_of(t_begin + 2 * kChunk, blk);

  int emit_left = emit_every, emit_k = 0;
  int stores_last = 0, stores_before = 0;  // store instructions issued after the last / the last but one request
  int tile_off = 0;
  for (int ti = t_begin; ti < t_end; ti += kChunk) {
    // this chunk's tile has landed; the next chunk's eight loads (and partials stored since this
    // tile was requested) may still be on their way
    wait_vm_all_but(stores_before + (ti + kChunk < t_end ? 8 : 0) + stores_last);
    const uint8_t *tile = wave_lds + tile_off;
    u32x4 kraw[4];
    u32x2 vt[4][2];
#pragma unroll
    for (int b = 0; b < 4; ++b) kraw[b] = *(const u32x4 *)(tile + b * 1024 + (k_rd ^ ((b & 1) ? 32u : 0u)));
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) vt[mt][pr] = lds_read_tr8(tile + pr * 2048 + (vt_rd ^ (uint32_t)(mt * 16)));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (ti + 2 * kChunk < t_end) {
      issue(tile_off, ti + 2 * kChunk, blk);
      if (ti + 3 * kChunk < t_end) pages_of(ti + 3 * kChunk, blk);
    }
    tile_off = kFp8TileBytes - tile_off;
    Frag8 kf[4][2], vf[4][2];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      fp8x8_to_bf16x8(kraw[b][0], kraw[b][1], kf[b][0].w);
      fp8x8_to_bf16x8(kraw[b][2], kraw[b][3], kf[b][1].w);
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) fp8x8_to_bf16x8(vt[mt][pr][0], vt[mt][pr][1], vf[mt][pr].w);
    const bool need_mask = (ti < lo_last) || (ti + kChunk > pos_first + 1);
    chunk_core<NT, false, false, false>(kf, vf, qf, ri, ti, need_mask, c2, m, lacc, acc, nullptr);
    stores_before = stores_last;
    stores_last = 0;
    if constexpr (!std::is_same<Emit, NoEmit>::value) {
      emit_left -= kChunk;
      if (emit_left == 0 && ti + kChunk < t_end) {  // (wave-uniform)
        stores_last = emit(emit_k++);
        emit_left = emit_every;
      }
    }
  }
}

// Finish a row tile: either normalise with the sink and store bf16 output (+lse), or store
// the partition's partial (m, l, acc) for the merge kernel.
//
// SINK_IN: the caller has the lane's sink (log2 units, -inf for none) in `sink_in` already;
// only where every row tile of a lane belongs to one query head (PAIR = false).
template <int NT, bool FP8, bool PAIR = false, bool SINK_IN = false>
__device__ __forceinline__ void finish(const AttnParams &p, const int s, const int kvh,
                                       const int row0, const int qlen, const int tq0,
                                       const bool direct, const int part, float (&m)[NT],
                                       f32x4 (&lacc)[NT], f32x4 (&acc)[NT][4],
                                       const float sink_in = 0.f) {
  static_assert(!(PAIR && SINK_IN), "head pairs spread a lane's tiles over two heads");
  const int lane = threadIdx.x & 63;
  const int i16 = lane & 15, g = lane >> 4;
  const int Hq = p.num_q_heads;
  const float vs = FP8 ? p.v_scale[PAIR ? kvh + (i16 >> 3) : kvh] : 1.0f;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const float l = lacc[nt][0];  // every lane of the row holds the full sum
    const int r = nt * 16 + i16;
    // (PAIR: one query token, the 16 rows are the 16 query heads of the two KV heads)
    const int t = PAIR ? tq0 : tq0 + (r >> 3);
    const int head = PAIR ? kvh * kGroup + r : kvh * kGroup + (r & 7);
    const bool valid = t < qlen;
    if (direct) {
      if (!valid) continue;
      const float sink2 = SINK_IN ? sink_in : (p.sinks ? p.sinks[head] * kLog2e : -INFINITY);
      const float M = fmaxf(m[nt], sink2);
      const float w = fast_exp2(m[nt] - M);
      const float den = l * w + fast_exp2(sink2 - M);
      const float inv = w * vs / den;
      uint16_t *o = p.out + ((size_t)(row0 + t) * Hq + head) * kHeadDim + 4 * g;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        u32x2 pk;
        pk[0] = pack_bf16(acc[nt][mt][0] * inv, acc[nt][mt][1] * inv);
        pk[1] = pack_bf16(acc[nt][mt][2] * inv, acc[nt][mt][3] * inv);
        *(u32x2 *)(o + 16 * mt) = pk;
      }
      if (p.lse && g == 0) p.lse[(size_t)(row0 + t) * Hq + head] = (M + __log2f(den)) * kLn2;
    } else {
      // Partials are laid out [row][partition][head]: the 8 heads of this wave are
      // neighbours, and the 64 heads of the workgroup form one contiguous 8 KiB block.
      const size_t idx = ((size_t)(s * p.ws_rows + t) * p.nparts_max + part) * Hq + head;
      if (valid && g == 0) {
        float2 ml;
        ml.x = l > 0.f ? m[nt] * kLn2 : -INFINITY;
        ml.y = l;
        *(float2 *)(p.ws_ml + idx * 2) = ml;
      }
      // the partition's own normalised output, fp16: half the workspace traffic of fp32
      // sums, and |o| <= max|v| whatever the softmax weights were
      const float inv_l = l > 0.f ? vs / l : 0.f;
      uint32_t w[4][2];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
        // (saturated to the fp16 range: a value entry beyond +-65504, which bf16 can hold, then
        // gives a bounded error in a sequence of several pieces, not an inf that the merge turns
        // into NaN)
        auto h = [&](const float x) { return (_Float16)__builtin_fminf(__builtin_fmaxf(x * inv_l, -65504.f), 65504.f); };
        const f16x2 h0 = {h(acc[nt][mt][0]), h(acc[nt][mt][1])};
        const f16x2 h1 = {h(acc[nt][mt][2]), h(acc[nt][mt][3])};
        w[mt][0] = __builtin_bit_cast(uint32_t, h0);
        w[mt][1] = __builtin_bit_cast(uint32_t, h1);
      }
      // A lane holds dims 16 mt + 4 g .. +3 of its row.  Swapping the odd 16-lane rows of
      // tile mt with the even rows of tile mt + 1 leaves every lane with 8 consecutive dims
      // (16 bytes): at (g & 1) * 16 + (g >> 1) * 8, from tiles {0, 1} and again from {2, 3}.
      // Executed by all lanes; only the stores are predicated.
#pragma unroll
      for (int mt = 0; mt < 4; mt += 2) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const auto r = __builtin_amdgcn_permlane16_swap(w[mt][k], w[mt + 1][k], false, false);
          w[mt][k] = r[0];
          w[mt + 1][k] = r[1];
        }
      }
      if (valid) {
        _Float16 *a = p.ws_acc + idx * kHeadDim + (g & 1) * 16 + (g >> 1) * 8;
        *(u32x4 *)a = u32x4{w[0][0], w[0][1], w[1][0], w[1][1]};
        *(u32x4 *)(a + 32) = u32x4{w[2][0], w[2][1], w[3][0], w[3][1]};
      }
    }
  }
}

// PRE: the operands are multiplied by `c2` (fp32 product, rounded to bf16 once) for
// chunk_step<.., PRE = true>.
template <int NT, bool PRE = false, bool PAIR = false>
__device__ __forceinline__ void load_q(const AttnParams &p, const int row0, const int qlen,
                                       const int tq0, const int kvh, const int pos0,
                                       Frag8 (&qf)[NT][2], RowInfo &ri, const float c2 = 1.0f) {
  const int lane = threadIdx.x & 63;
  const int i16 = lane & 15, g = lane >> 4;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int r = nt * 16 + i16;
    const int t = PAIR ? tq0 : tq0 + (r >> 3);
    const bool valid = t < qlen;
    const int tt = valid ? t : tq0;
    const uint16_t *qp = p.q + ((size_t)(row0 + tt) * p.num_q_heads + kvh * kGroup +
                                (PAIR ? r : (r & 7))) * kHeadDim + g * 16;
    qf[nt][0].u = valid ? *(const u32x4 *)qp : u32x4{0, 0, 0, 0};
    qf[nt][1].u = valid ? *(const u32x4 *)(qp + 8) : u32x4{0, 0, 0, 0};
    if constexpr (PRE) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t x = qf[nt][h].w[w];
          qf[nt][h].w[w] = pack_bf16(bf16_bits_to_f32(x & 0xffffu) * c2,
                                     __uint_as_float(x & 0xffff0000u) * c2);
        }
    }
  }
  ri.t_lane = PAIR ? tq0 : tq0 + (i16 >> 3);
  ri.tq0 = tq0;
  ri.qlen = qlen;
  ri.pos0 = pos0;
  ri.window = p.window;
}

// Work-item lookup shared by the split-KV kernel: the launch serves the compacted list of
// (sequence, partition) pairs of all sequences whose q_len lies in [qlen_lo, qlen_hi],
// enumerated sequence-major.  Item `w` is found by a wave-wide prefix sum over the
// per-sequence partition counts (64 sequences per pass).  Consecutive items go to
// consecutive workgroup ids, which the hardware deals round-robin to the 8 XCDs, so every
// XCD receives the same number of equal-sized items whatever the raggedness of the batch;
// ids past the end of the list are the only ones that exit without work.
struct WorkItem {
  int seq, part, nparts, row0, qlen, seq_len;
};

// Inclusive prefix sum over the 64 lanes with DPP adds (row shifts, then the row totals
// carried over with row_bcast): six dependent VALU ops instead of six LDS-crossbar
// permutes.  A lane whose DPP source is out of range, or whose row is masked off, adds
// the `old` operand, 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_add(const int v) {
  return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ int wave_inclusive_scan(int v, const int /*lane*/) {
  v = dpp_add<0x111, 0xf>(v);  // row_shr:1
  v = dpp_add<0x112, 0xf>(v);  // row_shr:2
  v = dpp_add<0x114, 0xf>(v);  // row_shr:4
  v = dpp_add<0x118, 0xf>(v);  // row_shr:8
  v = dpp_add<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}
// Sum over the 64 lanes, returned as a wave-uniform (scalar) value.  v must be >= 0.
__device__ __forceinline__ int wave_total(const int v) {
  return __builtin_amdgcn_readlane(wave_inclusive_scan(v, 0), 63);
}
__device__ __forceinline__ long long wave_total64(const long long v) {
  // three 22-bit limbs: each limb's 64-lane sum stays below 2^28
  const long long a = wave_total((int)(v & 0x3fffff));
  const long long b = wave_total((int)((v >> 22) & 0x3fffff));
  const long long c = wave_total((int)(v >> 44));
  return a + (b << 22) + (c << 44);
}
// Maximum over the 64 lanes of a value >= 0, wave-uniform (same DPP ladder as the scan; a lane
// without a source takes 0).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_max(const int v) {
  return max(v, __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ int wave_max(int v) {
  v = dpp_max<0x111, 0xf>(v);
  v = dpp_max<0x112, 0xf>(v);
  v = dpp_max<0x114, 0xf>(v);
  v = dpp_max<0x118, 0xf>(v);
  v = dpp_max<0x142, 0xa>(v);
  v = dpp_max<0x143, 0xc>(v);
  return __builtin_amdgcn_readlane(v, 63);
}
// a / b for wave-uniform a >= 0, b > 0: the 64-bit division expands to some hundred
// instructions, the 32-bit one to a third of that, and batches rarely need the former.
__device__ __forceinline__ long long uniform_div(const long long a, const long long b) {
  if (a < 0x7fffffffLL && b < 0x7fffffffLL) return (long long)((unsigned)a / (unsigned)b);
  return a / b;
}

// Per-lane view of one sequence for the planning passes: partitions are counted from the
// first visible page (kv_begin) to the end of the sequence.
struct SeqView {
  int span, row0, qlen, seq_len;
};

__device__ __forceinline__ SeqView view_seq(const AttnParams &p, const int s) {
  SeqView v{0, 0, 0, 0};
  if (s < p.num_seqs) {
    // (a length beyond the table row is a caller error; clamped, it cannot index past the row)
    v.seq_len = min(p.seq_lens[s], p.max_blocks_per_seq * kBlock);
    v.row0 = s;
    v.qlen = 1;
    if (p.cu_seqlens_q) {
      v.row0 = p.cu_seqlens_q[s];
      v.qlen = p.cu_seqlens_q[s + 1] - v.row0;
    }
    if (v.qlen >= p.qlen_lo && v.qlen <= p.qlen_hi && v.qlen <= p.ws_rows && v.seq_len >= v.qlen)
      v.span = v.seq_len - kv_begin(v.seq_len, v.qlen, p.window);
  }
  return v;
}

__device__ __forceinline__ int num_partitions(const AttnParams &p, const int span, const int P) {
  return min((span + P - 1) / P, p.nparts_max);
}

// Partition size of this launch.  Fixed when the caller gave one.  Otherwise every wave
// derives the same value from the batch itself.  With T = workgroups the device holds at
// once: if the whole batch fits one device fill with partitions no longer than the cap,
// take the smallest multiple of 64 (>= the planning minimum that sized the workspace)
// whose exact item count is <= T, so every workgroup is resident from the start and no
// second, partly filled round follows; otherwise size the partition for about three fills
// of equal items (two fills balance ragged batches badly, many small items pay the
// per-item prologue too often), between a floor and the cap.  `first` is the view of sequences 0..63 (one per lane), which the
// caller has loaded already.
__device__ __forceinline__ int effective_partition(const AttnParams &p, const SeqView &first) {
  if (!p.dynamic_partition) return p.partition;
  const int lane = threadIdx.x & 63;
  long long total = first.span;
  int longest = first.span;
  int active = __popcll(__ballot(first.span > 0));
  for (int s0 = 64; s0 < p.num_seqs; s0 += 64) {
    const SeqView v = view_seq(p, s0 + lane);
    total += v.span;
    longest = max(longest, v.span);
    active += __popcll(__ballot(v.span > 0));
  }
  total = wave_total64(total);
  longest = wave_max(longest);
  const long long T = max(p.target_items, 1);
  // (every value below is the same in all lanes and lives in scalar registers, and so does
  // everything derived from the partition)
  // Smallest multiple of 64 (>= the planning minimum, < the cap) whose exact item count
  // is <= Tx, or 0 if there is none.  Two sizes are known to fit: the pessimistic bound
  // total / (Tx - active) (every sequence may add one short item), and the longest span,
  // which makes every sequence a single item (the only way when active == Tx).  The exact
  // count falls as the partition grows, so the smallest fitting size below the better of
  // the two is found by bisection (a handful of counts).
  auto single_fill = [&](const long long Tx) -> int {
    if (active > Tx) return 0;
    long long hi = ((long long)longest + 63) / 64 * 64;
    if (active < Tx)
      hi = min(hi, (uniform_div(total + (Tx - active) - 1, Tx - active) + 63) / 64 * 64);
    hi = max(hi, (long long)p.partition);
    if (hi >= kDynPartitionCap) return 0;
    int lo_i = p.partition / 64, hi_i = (int)hi / 64 - 1, P = (int)hi;
    while (lo_i <= hi_i) {
      const int mid = (lo_i + hi_i) >> 1, Pc = mid * 64;
      int items = num_partitions(p, first.span, Pc);
      for (int s0 = 64; s0 < p.num_seqs; s0 += 64)
        items += num_partitions(p, view_seq(p, s0 + lane).span, Pc);
      if (wave_total64(items) <= Tx) {
        P = Pc;
        hi_i = mid - 1;
      } else {
        lo_i = mid + 1;
      }
    }
    return P;
  };
  // one workgroup per CU if the batch is small enough for that, else one device fill
  if (p.target_items_lo < T) {
    const int P = single_fill(max(p.target_items_lo, 1));
    if (P) return P;
  }
  if (const int P = single_fill(T)) return P;
  // More than one fill.  At least one sequence per CU and none longer than the cap: every
  // sequence is one item (no partials, no merge); the dispatcher evens out ragged lengths
  // over the rounds.
  const int whole = (longest + 63) / 64 * 64;
  if (active >= p.target_items_lo && whole <= kDynPartitionCap) return max(whole, p.partition);
  // Nearly uniform lengths (longest within a quarter of the mean): equal pieces of every
  // sequence, as few as the cap allows; there is no raggedness for small items to even out,
  // and every item pays a prologue and a partial.
  if ((long long)longest * active * 4 <= total * 5) {
    const int pieces = (longest + kDynPartitionCap - 1) / kDynPartitionCap;
    return max(((longest + pieces - 1) / pieces + 63) / 64 * 64, p.partition);
  }
  // Ragged: aim at about three fills of equal items, within [floor, cap]
  return (int)min((long long)kDynPartitionCap,
                  max((long long)kDynPartitionFloor, (uniform_div(total, 3 * T) + 63) / 64 * 64));
}

// Partition size of this launch: from the plan header when a plan kernel ran, else derived
// here.  With a plan, `w` past the end of the item list is known at once.
__device__ __forceinline__ bool planned_out(const AttnParams &p, const int w) {
  return p.plan && w >= p.plan[1];
}

// Finds item `w` of the compacted list and the partition size it was built with.
__device__ __forceinline__ bool find_work_item(const AttnParams &p, const int w, int &P,
                                               WorkItem &it) {
  const int lane = threadIdx.x & 63;
  const SeqView first = view_seq(p, lane);
  P = p.plan ? p.plan[0] : effective_partition(p, first);
  int base = 0;
  for (int s0 = 0; s0 < p.num_seqs; s0 += 64) {
    const SeqView v = s0 == 0 ? first : view_seq(p, s0 + lane);
    const int n = num_partitions(p, v.span, P);
    const int incl = wave_inclusive_scan(n, lane);
    const int total = __builtin_amdgcn_readlane(incl, 63);
    if (w < base + total) {
      const unsigned long long hit = __ballot(base + incl > w);
      const int idx = __builtin_ctzll(hit);
      it.seq = s0 + idx;
      it.nparts = __builtin_amdgcn_readlane(n, idx);
      it.part = w - (base + __builtin_amdgcn_readlane(incl, idx) - it.nparts);
      it.row0 = __builtin_amdgcn_readlane(v.row0, idx);
      it.qlen = __builtin_amdgcn_readlane(v.qlen, idx);
      it.seq_len = __builtin_amdgcn_readlane(v.seq_len, idx);
      return true;
    }
    base += total;
  }
  return false;
}

// ---------------------------------------------------------------------------------------
// Plan kernel (one wave).  The host sizes the split-KV grid from max_kv_len alone, so on
// ragged batches most of that grid has nothing to do, and a workgroup that has to scan
// seq_lens to find that out still costs a dispatch, a slot and ~2 us.  When the bound is
// large the library runs this kernel first: it writes {partition, number of items} to the
// head of the workspace, and every surplus workgroup then leaves after one scalar load.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void plan_kernel(const AttnParams p, int32_t *plan_out) {
  const int lane = threadIdx.x & 63;
  const SeqView first = view_seq(p, lane);
  const int P = effective_partition(p, first);
  long long items = num_partitions(p, first.span, P);
  for (int s0 = 64; s0 < p.num_seqs; s0 += 64)
    items += num_partitions(p, view_seq(p, s0 + lane).span, P);
  items = wave_total64(items);
  if (lane == 0) {
    plan_out[0] = P;
    plan_out[1] = (int32_t)items;
  }
}

// One work item: wave `wave` of the workgroup attends the rows of KV head `kvh` over
// partition it.part (P tokens) of sequence it.seq and writes the output or the partial.
template <int NT, bool FP8, bool PAIR = false, bool DMA = false>
__device__ __forceinline__ void splitkv_item(const AttnParams &p, const WorkItem &it, const int P,
                                             const int kvh, const int wave, uint8_t *lds,
                                             const FirstPages &first = FirstPages{},
                                             const int tq0 = 0) {
  const int s = it.seq, part = it.part, nparts = it.nparts;
  const int row0 = it.row0, qlen = it.qlen, L = it.seq_len;
  const int kb = kv_begin(L, qlen, p.window);
  const int t0 = kb + part * P;
  const int t1 = min(t0 + P, L);
  const int pos0 = L - qlen;
  const int lo_last = p.window > 0 ? max(0, L - p.window) : 0;

  Frag8 qf[NT][2];
  RowInfo ri;
  if (tq0 >= qlen) return;  // (a row group past the sequence's rows)
  load_q<NT, false, PAIR>(p, row0, qlen, tq0, kvh, pos0, qf, ri);
  float m[NT];
  f32x4 lacc[NT], acc[NT][4];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    m[nt] = kNegBig;
    lacc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  if constexpr (DMA)
    attend_dma<NT>(p, s, kvh, t0, t1, L, pos0, lo_last, qf, ri, lds + wave * kWaveDmaBytes, m, lacc, acc, first);
  else
    attend<NT, FP8, PAIR>(p, s, kvh, t0, t1, L, pos0, lo_last, qf, ri, lds + wave * kWaveLdsBytes,
                          m, lacc, acc, first);
  finish<NT, FP8, PAIR>(p, s, kvh, row0, qlen, tq0, nparts == 1, part, m, lacc, acc);
}

// ---------------------------------------------------------------------------------------
// Split-KV kernel.  grid = (num_seqs * nparts_max, Hkv / WAVES); workgroup blockIdx.x takes
// work item blockIdx.x (see find_work_item) and wave w of it owns KV head
// blockIdx.y*WAVES + w, so the workgroup as a whole streams whole 16-token pages (all KV
// heads) of its partition.
// ---------------------------------------------------------------------------------------
//
// RS > 1 (q_len beyond one wave's rows): RS waves share a KV head, wave w taking the query
// tokens [8 (w % RS), +8) of the sequence; the workgroup then covers WAVES / RS KV heads and
// the grid's y dimension grows by RS.  Both waves load the head's K/V (the second from cache).
//
// PAIR (fp8 decode rows): every wave owns two neighbouring KV heads, see chunk_step.
//
// DMA (bf16 cache): the chunks come in by direct global -> LDS loads (attend_dma); 16 KiB of LDS
// per wave, i.e. one 8-wave workgroup per CU.
template <int NT, bool FP8, int WAVES, int RS = 1, bool PAIR = false, bool DMA = false>
__global__ __launch_bounds__(WAVES * 64, ((NT == 1 && !DMA) ? 4 : 2)) void splitkv_kernel(const AttnParams p) {
  static_assert(RS == 1 || (NT == 4 && WAVES % RS == 0), "row groups are 8 tokens = four tiles");
  static_assert(!PAIR || RS == 1, "head pairs have one row group");
  static_assert(!DMA || (!FP8 && RS == 1), "direct loads: bf16 cache, one row group");
  __shared__ __align__(1024) uint8_t lds[WAVES * (DMA ? kWaveDmaBytes : kWaveLdsBytes)];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = (blockIdx.y * (WAVES / RS) + wave / RS) * (PAIR ? 2 : 1);
  const int tq0 = (wave % RS) * (NT * 16 / kGroup);
  if (p.nparts_max == 1) {
    // Every sequence is a single item (short spans: sliding-window layers, short contexts):
    // workgroup w serves sequence w, found with scalar loads alone; sequences of another
    // q_len class leave at once.
    const SeqView v = view_seq(p, blockIdx.x);
    // (every sequence one partition: a merge called by itself afterwards finds nothing to do)
    if (p.plan_slot && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) p.plan_slot[0] = 1 << 30;
    if (v.span <= 0) return;
    WorkItem it;
    it.seq = blockIdx.x;
    it.part = 0;
    it.nparts = 1;
    it.row0 = v.row0;
    it.qlen = v.qlen;
    it.seq_len = v.seq_len;
    splitkv_item<NT, FP8, PAIR, DMA>(p, it, 1 << 30, kvh, wave, lds, FirstPages{}, tq0);
    return;
  }
  if (planned_out(p, blockIdx.x)) return;
  // One wave looks the work item up and hands it to the others through LDS: the lookup is
  // several hundred instructions, and eight waves doing it side by side on every CU at the
  // start of the launch would spend microseconds of issue slots before the first K/V load.
  __shared__ int item_lds[8];
  if (wave == 0) {
    int P0 = 0;
    WorkItem w{};
    const bool found = find_work_item(p, blockIdx.x, P0, w);
    if ((threadIdx.x & 63) == 0) {
      item_lds[0] = found ? P0 : 0;
      item_lds[1] = w.seq;
      item_lds[2] = w.part;
      item_lds[3] = w.nparts;
      item_lds[4] = w.row0;
      item_lds[5] = w.qlen;
      item_lds[6] = w.seq_len;
    }
  }
  __syncthreads();
  const int P = __builtin_amdgcn_readfirstlane(item_lds[0]);
  if (P == 0) return;  // past the end of the item list
  WorkItem it;
  it.seq = __builtin_amdgcn_readfirstlane(item_lds[1]);
  it.part = __builtin_amdgcn_readfirstlane(item_lds[2]);
  it.nparts = __builtin_amdgcn_readfirstlane(item_lds[3]);
  it.row0 = __builtin_amdgcn_readfirstlane(item_lds[4]);
  it.qlen = __builtin_amdgcn_readfirstlane(item_lds[5]);
  it.seq_len = __builtin_amdgcn_readfirstlane(item_lds[6]);
  // the merge launch that follows reads the partition from here instead of re-deriving it
  if (!p.plan && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) p.plan_slot[0] = P;
  splitkv_item<NT, FP8, PAIR, DMA>(p, it, P, kvh, wave, lds, FirstPages{}, tq0);
}

// The same for a decode launch whose items the host has listed (q_len 1, row = sequence):
// no scan, no hand-over through LDS.
__device__ __forceinline__ WorkItem table_item(const AttnParams &p, const ItemTable &tab,
                                               const int w, const int P) {
  const unsigned long long e = tab.e[w];
  WorkItem it;
  it.seq = (int)(e & 0xffffu);
  it.part = (int)((e >> 16) & 0xffffu);
  it.seq_len = min((int)(e >> 32), p.max_blocks_per_seq * kBlock);
  it.row0 = it.seq;
  it.qlen = 1;
  it.nparts = num_partitions(p, it.seq_len - kv_begin(it.seq_len, 1, p.window), P);
  return it;
}

template <int NT, bool FP8, int WAVES, bool PAIR = false, bool DMA = false>
__global__ __launch_bounds__(WAVES * 64, ((NT == 1 && !DMA) ? 4 : 2)) void splitkv_table_kernel(
    const AttnParams p, const ItemTable tab) {
  __shared__ __align__(1024) uint8_t lds[WAVES * (DMA ? kWaveDmaBytes : kWaveLdsBytes)];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = (blockIdx.y * WAVES + wave) * (PAIR ? 2 : 1);
  if ((int)blockIdx.x >= tab.n) return;
  const int P = p.partition;
  const WorkItem it = table_item(p, tab, blockIdx.x, P);
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) p.plan_slot[0] = P;
  FirstPages first;  // (read element by element: a pointer into the argument would make the
  first.have = tab.has_blk;  // compiler copy the whole list into private memory)
#pragma unroll
  for (int b = 0; b < 4; ++b) first.id[b] = tab.blk[blockIdx.x][b];
  splitkv_item<NT, FP8, PAIR, DMA>(p, it, P, kvh, wave, lds, first);
}

// ---------------------------------------------------------------------------------------
// Even split.  One workgroup per work item leaves much of the device idle on long launches:
// every item pays a dispatch, the item lookup, the loads of Q and of its first page ids and, at
// its end, the hardware's wait for the partial stores before the slot is handed on (about
// 10 us next to 42 us of streaming for a 512-key item of five query rows, with nothing of the
// CU in flight meanwhile where one workgroup fits a CU), and a batch of ragged sequences cut
// into one device fill of items leaves a third of the slots idle behind the longest items.
// Here the launch's units - 64-key chunks (run-time partition) or partitions of the caller's
// size - are laid out sequence after sequence and cut into gridDim.x equal, contiguous ranges
// of `q` units: workgroup b walks units [b q, (b + 1) q), from the middle of one sequence
// through whole sequences into the start of another.  Q is loaded once per sequence visited
// and the page-id prefetch runs through.  Equal unit counts are equal work.
//
// What a workgroup holds of one sequence is one PIECE: it carries (m, l, acc) through the
// piece's units - the rescaling of the online softmax IS the log-sum-exp merge of consecutive
// partitions, done in registers - and stores one partial where its range leaves the sequence.
// The caller's partition size is then the grid on which ranges may be cut, not a number of
// round trips through memory: on this machine stores trickling into a saturated stream of
// loads are dear out of all proportion (a plain gather of config 5's pages at 6.9 TB/s drops
// to 4.9 TB/s when 4 % of its traffic is partial stores), so a partial per 512 keys costs a
// quarter of the run time.  p.store_every_partition (a measurement aid) restores that form:
// a partial per partition, all of them merged by the merge kernel.
// The pieces of a sequence have no common size.  Piece index = workgroup id - id of the
// workgroup holding the sequence's first unit; that workgroup records the sequence's number
// of pieces in p.seq_parts for the merge, and the plan slot receives kEvenFlag | q.  With a
// run-time partition q >= kEvenMinChunks, so a sequence of n chunks has at most
// ceil(n / kEvenMinChunks) + 1 pieces, which is what the workspace is sized for.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ SeqView view_seq_uniform(const AttnParams &p, const int s) {
  // (s is wave-uniform: the loads go through the scalar unit)
  SeqView v{0, 0, 0, 0};
  if (s < p.num_seqs) {
    v.seq_len = min(as_constant(p.seq_lens)[s], p.max_blocks_per_seq * kBlock);
    v.row0 = s;
    v.qlen = 1;
    if (p.cu_seqlens_q) {
      const const_i32_ptr cu = as_constant(p.cu_seqlens_q);
      v.row0 = cu[s];
      v.qlen = cu[s + 1] - v.row0;
    }
    if (v.qlen >= p.qlen_lo && v.qlen <= p.qlen_hi && v.qlen <= p.ws_rows && v.seq_len >= v.qlen)
      v.span = v.seq_len - kv_begin(v.seq_len, v.qlen, p.window);
  }
  return v;
}

// Units of a sequence in an even split: chunks, or partitions of the caller's size.
__device__ __forceinline__ int even_units(const AttnParams &p, const int span) {
  return p.dynamic_partition ? (span + kChunk - 1) / kChunk : num_partitions(p, span, p.partition);
}

// Quota and start of workgroup `b` of `G`: q = units per workgroup, (seq, unit) = where its
// range begins.  False when the range is empty.  Executed by one wave.
__device__ __forceinline__ bool even_find_start(const AttnParams &p, const int b, const int G,
                                                int &q, int &seq, int &unit) {
  const int lane = threadIdx.x & 63;
  long long C = 0;
  for (int s0 = 0; s0 < p.num_seqs; s0 += 64) C += even_units(p, view_seq(p, s0 + lane).span);
  C = wave_total64(C);
  q = (int)max(uniform_div(C + G - 1, G), (long long)(p.dynamic_partition ? kEvenMinChunks : 1));
  const long long start = (long long)b * q;
  if (start >= C) return false;
  long long base = 0;
  for (int s0 = 0; s0 < p.num_seqs; s0 += 64) {
    const int n = even_units(p, view_seq(p, s0 + lane).span);
    const int incl = wave_inclusive_scan(n, lane);
    const int total = __builtin_amdgcn_readlane(incl, 63);
    if (start < base + total) {
      const int rel = (int)(start - base);
      const int idx = __builtin_ctzll(__ballot(incl > rel));
      seq = s0 + idx;
      unit = rel - (__builtin_amdgcn_readlane(incl, idx) - __builtin_amdgcn_readlane(n, idx));
      return true;
    }
    base += total;
  }
  return false;
}

// (two waves per SIMD, i.e. all 256 registers: eight waves per CU; the head-pair kernel moves
// half the bytes per wave and load, and keeps sixteen)
template <int NT, bool FP8, int WAVES, bool PAIR = false, bool DMA = false>
__global__ __launch_bounds__(WAVES * 64, ((PAIR && !DMA) ? 4 : 2)) void splitkv_even_kernel(const AttnParams p,
                                                                                          const EvenTable tab) {
  constexpr int kWaveBytes = !DMA ? kWaveLdsBytes : PAIR ? kWavePairDmaBytes : FP8 ? kWaveFp8DmaBytes : kWaveDmaBytes;
  __shared__ __align__(1024) uint8_t lds[WAVES * kWaveBytes];
  __shared__ int start_lds[4];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kvh = (blockIdx.y * WAVES + wave) * (PAIR ? 2 : 1);
  const int b = blockIdx.x;
  const bool dyn = p.dynamic_partition != 0;
  int q, s, u;
  if (tab.n > 0) {
    if (b >= tab.n) return;
    q = tab.q;
    const uint32_t e = tab.start[b];
    s = (int)(e & 0xffffu);
    u = (int)(e >> 16);
  } else {
    if (wave == 0) {
      int q0 = 0, s0 = 0, u0 = 0;
      const bool found = even_find_start(p, b, gridDim.x, q0, s0, u0);
      if ((threadIdx.x & 63) == 0) {
        start_lds[0] = found ? q0 : 0;
        start_lds[1] = s0;
        start_lds[2] = u0;
      }
    }
    __syncthreads();
    q = __builtin_amdgcn_readfirstlane(start_lds[0]);
    if (q == 0) return;
    s = __builtin_amdgcn_readfirstlane(start_lds[1]);
    u = __builtin_amdgcn_readfirstlane(start_lds[2]);
  }
  // pieces (one partial per workgroup and sequence), or a partial per partition of the caller's
  const bool pieces = dyn || !p.store_every_partition;
  // the merge that follows reads the mode (and, with a partial per partition, its size) from here
  if (b == 0 && blockIdx.y == 0 && threadIdx.x == 0) p.plan_slot[0] = pieces ? (kEvenFlag | q) : p.partition;
  const int U = dyn ? kChunk : p.partition;  // keys per unit
  uint8_t *wave_lds = lds + wave * kWaveBytes;
  int rem = q;
  bool first_seq = true;
  SeqView v = view_seq_uniform(p, s);
  while (rem > 0 && s < p.num_seqs) {
    const int n_s = even_units(p, v.span);
    const int n_here = min(rem, n_s - u);
    const int s_now = s, u_now = u;
    const SeqView v_now = v;
    // next sequence of this class (its lengths are requested before this one is walked)
    rem -= n_here;
    u = 0;
    do {
      ++s;
      v = view_seq_uniform(p, s);
    } while (s < p.num_seqs && v.span <= 0);
    if (n_here <= 0) continue;  // (only a malformed start: the range begins past a sequence's end)
    const int L = v_now.seq_len, qlen = v_now.qlen, row0 = v_now.row0;
    const int kb = kv_begin(L, qlen, p.window);
    const int t0 = kb + u_now * U;
    const int t1 = min(kb + (u_now + n_here) * U, L);
    const int pos0 = L - qlen;
    const int lo_last = p.window > 0 ? max(0, L - p.window) : 0;
    // the piece (run-time partition) or the first partition (caller's) and the sequence's count
    int part, nparts;
    if (pieces) {
      // units before this sequence: (b q + units of the range used up so far) - u_now
      part = first_seq ? (u_now + q - 1) / q : 0;
      // first workgroup of the sequence holds its unit 0: the sequence starts `off` units into it
      const int off = first_seq ? (q - (u_now % q)) % q : q - (rem + n_here);
      nparts = (off + n_s - 1) / q + 1;
      if (part == 0 && wave == 0 && blockIdx.y == 0 && (threadIdx.x & 63) == 0) p.seq_parts[s_now] = nparts;
    } else {
      part = u_now;
      nparts = n_s;
    }
    first_seq = false;
    Frag8 qf[NT][2];
    RowInfo ri;
    load_q<NT, false, PAIR>(p, row0, qlen, 0, kvh, pos0, qf, ri);
    float m[NT];
    f32x4 lacc[NT], acc[NT][4];
    auto reset = [&]() {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        m[nt] = kNegBig;
        lacc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
    };
    reset();
    const bool direct = nparts == 1;
    auto emit = [&](const int k) {
      finish<NT, FP8, PAIR>(p, s_now, kvh, row0, qlen, 0, false, part + k, m, lacc, acc);
      reset();
      // finish() stores (m, l) and two 16-byte pieces per lane for every tile that holds a row
      return 3 * min(NT, (qlen + 1) / 2);
    };
    if constexpr (DMA && PAIR)
      attend_dma_pair(p, s_now, kvh, t0, t1, L, pos0, lo_last, qf, ri, wave_lds, m, lacc, acc, pieces ? 0 : U, emit);
    else if constexpr (DMA && FP8)
      attend_dma_fp8<NT>(p, s_now, kvh, t0, t1, L, pos0, lo_last, qf, ri, wave_lds, m, lacc, acc, pieces ? 0 : U, emit);
    else if constexpr (DMA)
      attend_dma<NT>(p, s_now, kvh, t0, t1, L, pos0, lo_last, qf, ri, wave_lds, m, lacc, acc, FirstPages{},
                     pieces ? 0 : U, emit);
    else
      attend<NT, FP8, PAIR>(p, s_now, kvh, t0, t1, L, pos0, lo_last, qf, ri, wave_lds, m, lacc, acc,
                            FirstPages{}, pieces ? 0 : U, emit);
    finish<NT, FP8, PAIR>(p, s_now, kvh, row0, qlen, 0, direct, pieces ? part : part + n_here - 1, m, lacc, acc);
  }
}

// ---------------------------------------------------------------------------------------
// Short-span kernel: one wave per 64-token chunk.  When no sequence spans more than 8 chunks
// (sliding-window layers, short contexts) a sequence is too short to be worth partitioning
// across workgroups, and one wave walking its 2-3 chunks one after the other is pure latency.
// Here a workgroup owns one (sequence, KV head) and its 8 waves take one chunk each, all in
// flight at once; the eight (m, l, acc) partials meet in LDS (each wave's V staging area is
// reused for its fp32 accumulators) and the 512 threads combine them with the sink and write
// the output.  grid = (num_seqs, Hkv); sequences of another q_len class leave at once.
//
// The same kernel serves small batches of longer sequences (nparts_max > 1): the sequences
// are cut into partitions of 8 chunks, a workgroup owns one (sequence, partition, KV head),
// found by the same scan as the split-KV kernel's work items, and writes the partition's
// (m, l) and normalised output to the workspace for the merge kernel.  The host takes this
// path when all workgroups are resident at once, so that every chunk of the batch is in
// flight from the start and the call lasts a few memory latencies, whatever the lengths.
// grid = (bound on the items, Hkv).
// ---------------------------------------------------------------------------------------
constexpr int kShortWaves = 8;
static_assert(kShortSpanMax == kShortWaves * kChunk, "one chunk per wave");

template <int NT, bool FP8>
__device__ __forceinline__ void shortspan_body(const AttnParams &p, const ItemTable *tab) {
  constexpr int kRows = NT * 16;
  constexpr int kPartBytes = kRows * kHeadDim * 4;  // one wave's fp32 accumulators
  constexpr int kWaveBytes = kPartBytes > kWaveLdsBytes ? kPartBytes : kWaveLdsBytes;
  __shared__ __align__(16) uint8_t lds[kShortWaves * kWaveBytes];
  __shared__ float ml_lds[kShortWaves][kRows][2];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int kvh = blockIdx.y;
  int s = blockIdx.x, part = 0, nparts = 1, L, qlen, row0;
  if (p.nparts_max == 1) {
    const SeqView v = view_seq(p, s);
    if (p.plan_slot && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) p.plan_slot[0] = 1 << 30;
    if (v.span <= 0) return;  // not of this class, or malformed: the whole workgroup leaves
    L = v.seq_len, qlen = v.qlen, row0 = v.row0;
  } else {
    // partitions of kShortSpanMax keys (the host set p.partition to that): the item comes
    // from the host's list, or every wave looks it up for itself (there is nothing else to
    // do yet and no barrier to wait at)
    WorkItem it;
    if (tab) {
      if ((int)blockIdx.x >= tab->n) return;
      it = table_item(p, *tab, blockIdx.x, kShortSpanMax);
    } else {
      int P;
      if (!find_work_item(p, blockIdx.x, P, it)) return;
    }
    s = it.seq, part = it.part, nparts = it.nparts;
    L = it.seq_len, qlen = it.qlen, row0 = it.row0;
    // the partition this launch ran with, for a merge that is called by itself afterwards
    if (p.plan_slot && blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) p.plan_slot[0] = kShortSpanMax;
  }
  const int pos0 = L - qlen;
  const int lo_last = p.window > 0 ? max(0, L - p.window) : 0;
  const int tb = kv_begin(L, qlen, p.window) + part * kShortSpanMax;  // this workgroup's keys
  const int te = min(tb + kShortSpanMax, L);
  const int nw = min(kShortWaves, (te - tb + kChunk - 1) / kChunk);  // waves with a chunk
  const int t0 = tb + wave * kChunk;
  if (wave < nw) {
    Frag8 qf[NT][2];
    RowInfo ri;
    load_q<NT>(p, row0, qlen, 0, kvh, pos0, qf, ri);
    float m[NT];
    f32x4 lacc[NT], acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      m[nt] = kNegBig;
      lacc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    uint8_t *mine = lds + wave * kWaveBytes;
    attend<NT, FP8>(p, s, kvh, t0, min(t0 + kChunk, te), L, pos0, lo_last, qf, ri, mine, m, lacc, acc);
    // the V tile is consumed: the same bytes now carry this wave's accumulators, row-major
    float *part = reinterpret_cast<float *>(mine);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
        *(f32x4 *)(part + (nt * 16 + i16) * kHeadDim + 16 * mt + 4 * g) = acc[nt][mt];
      if (g == 0) {
        ml_lds[wave][nt * 16 + i16][0] = m[nt];
        ml_lds[wave][nt * 16 + i16][1] = lacc[nt][0];
      }
    }
  }
  __syncthreads();
  // combine: 32 threads per row, two dims each
  const float vs = FP8 ? p.v_scale[kvh] : 1.0f;
  const int d2 = (tid & 31) * 2;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int r = nt * 16 + (tid >> 5);
    const int t = r >> 3;
    if (t >= qlen) continue;
    const int head = kvh * kGroup + (r & 7);
    if (nparts > 1) {
      // one of several partitions: its (m, l) and normalised output go to the workspace in
      // the split-KV kernel's layout, for the same merge
      float M = kNegBig;
      for (int w = 0; w < nw; ++w) M = fmaxf(M, ml_lds[w][r][0]);
      float l = 0.f, o0 = 0.f, o1 = 0.f;
      for (int w = 0; w < nw; ++w) {
        const float wgt = fast_exp2(ml_lds[w][r][0] - M);
        l += wgt * ml_lds[w][r][1];
        const float2 a = *(const float2 *)(lds + w * kWaveBytes + ((size_t)r * kHeadDim + d2) * 4);
        o0 += wgt * a.x;
        o1 += wgt * a.y;
      }
      const size_t idx = ((size_t)(s * p.ws_rows + t) * p.nparts_max + part) * p.num_q_heads + head;
      if (d2 == 0) *(float2 *)(p.ws_ml + idx * 2) = make_float2(l > 0.f ? M * kLn2 : -INFINITY, l);
      const float inv_l = l > 0.f ? vs / l : 0.f;
      typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
      *(f16x2 *)(p.ws_acc + idx * kHeadDim + d2) = f16x2{(_Float16)(o0 * inv_l), (_Float16)(o1 * inv_l)};
      continue;
    }
    const float sink2 = p.sinks ? p.sinks[head] * kLog2e : -INFINITY;
    float M = sink2;
    for (int w = 0; w < nw; ++w) M = fmaxf(M, ml_lds[w][r][0]);
    float den = fast_exp2(sink2 - M), o0 = 0.f, o1 = 0.f;
    for (int w = 0; w < nw; ++w) {
      const float wgt = fast_exp2(ml_lds[w][r][0] - M);
      den += wgt * ml_lds[w][r][1];
      const float2 a = *(const float2 *)(lds + w * kWaveBytes + ((size_t)r * kHeadDim + d2) * 4);
      o0 += wgt * a.x;
      o1 += wgt * a.y;
    }
    const float inv = vs / den;
    const size_t orow = (size_t)(row0 + t) * p.num_q_heads + head;
    *(uint32_t *)(p.out + orow * kHeadDim + d2) = pack_bf16(o0 * inv, o1 * inv);
    if (p.lse && d2 == 0) p.lse[orow] = (M + __log2f(den)) * kLn2;
  }
}

template <int NT, bool FP8>
__global__ __launch_bounds__(kShortWaves * 64, (NT == 1 ? 4 : 2)) void shortspan_kernel(const AttnParams p) {
  shortspan_body<NT, FP8>(p, nullptr);
}
template <int NT, bool FP8>
__global__ __launch_bounds__(kShortWaves * 64, (NT == 1 ? 4 : 2)) void shortspan_table_kernel(
    const AttnParams p, const ItemTable tab) {
  shortspan_body<NT, FP8>(p, &tab);
}

// ---------------------------------------------------------------------------------------
// Prefill kernel for long query chunks (q_len > 6): the MFMA-bound path.
//
// A workgroup of 4 waves owns 32 consecutive query tokens of one sequence for one KV head:
// 256 (token, head) rows, 64 per wave (four 16-row tiles).  It walks the keys its rows can
// see in 64-token chunks; each chunk's K and V (one KV head: 8 KiB each) are fetched from
// the paged cache ONCE per workgroup into a double-buffered LDS tile (rows padded to 144 B,
// fp8 widened on the way in) while the previous chunk is being consumed, and every wave
// reads its K operands (ds_read_b128) and V^T operands (ds_read_b64_tr_b16) from there.
//
// grid.x = Hkv * items with the KV head as the fastest index: workgroup ids are dealt
// round-robin to the 8 XCDs, so with 8 KV heads every XCD serves a single KV head and the
// K/V stream of a sequence is fetched into that XCD's L2 once for all its query tiles.
// Items = 32-token tiles of the sequences of this class, compacted by a prefix scan; within
// each batch of 64 sequences the longest come first, and within a sequence the latest
// (heaviest) tile comes first, so the long-running workgroups start early.
// ---------------------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void pf_gptr_t;
typedef __attribute__((address_space(3))) void pf_lptr_t;
constexpr int kPfWaves = 4;
constexpr int kPfWaveTok = 8;                     // query tokens per wave (x 8 heads = 64 rows)
constexpr int kPfTok = kPfWaves * kPfWaveTok;     // query tokens per workgroup
// Row strides of the LDS tiles.  K is read 16 bytes per lane by 16 lanes at a time, one row
// each: 144 B (36 banks) sends them to 16 distinct 4-bank groups.  V^T is read 8 bytes per
// lane by 32 lanes at a time, 8 rows x 32 B: that wants the rows 8 banks apart modulo 64,
// i.e. a stride of 8 x odd banks: 160 B.  (With 144 B rows 0 and 7 share banks.)
constexpr int kPfKRowBytes = 144;
constexpr int kPfVRowBytes = 160;
constexpr int kPfKTileBytes = kChunk * kPfKRowBytes;  // one 64-token K tile of one KV head
constexpr int kPfVTileBytes = kChunk * kPfVRowBytes;  // one 64-token V tile

__device__ __forceinline__ bool find_prefill_item(const AttnParams &p, const int w, int &seq,
                                                  int &tile, int &row0, int &qlen, int &seq_len) {
  const int lane = threadIdx.x & 63;
  int base = 0;
  for (int s0 = 0; s0 < p.num_seqs; s0 += 64) {
    const int s = s0 + lane;
    int n = 0, r0 = 0, ql = 0, L = 0;
    if (s < p.num_seqs) {
      L = min(p.seq_lens[s], p.max_blocks_per_seq * kBlock);
      r0 = p.cu_seqlens_q[s];
      ql = p.cu_seqlens_q[s + 1] - r0;
      if (ql >= p.qlen_lo && ql <= p.qlen_hi && L >= ql) n = (ql + kPfTok - 1) / kPfTok;
    }
    // Longest sequences first within the batch of 64 (their tiles walk the most keys):
    // rank by key length, then let lane r speak for the sequence of rank r.
    const int key = n > 0 ? L : -1;
    int rank = 0;
#pragma unroll
    for (int j = 0; j < 64; ++j) {
      const int kj = __builtin_amdgcn_readlane(key, j);
      rank += (kj > key || (kj == key && j < lane)) ? 1 : 0;
    }
    const int n_sorted = __builtin_amdgcn_ds_permute(rank << 2, n);
    const int lane_sorted = __builtin_amdgcn_ds_permute(rank << 2, lane);
    const int incl = wave_inclusive_scan(n_sorted, lane);
    const int total = __builtin_amdgcn_readlane(incl, 63);
    if (w < base + total) {
      const unsigned long long hit = __ballot(base + incl > w);
      const int pos = __builtin_ctzll(hit);
      const int idx = __builtin_amdgcn_readlane(lane_sorted, pos);
      const int nt = __builtin_amdgcn_readlane(n, idx);
      seq = s0 + idx;
      tile = nt - 1 - (w - (base + __builtin_amdgcn_readlane(incl, pos) - nt));
      row0 = __builtin_amdgcn_readlane(r0, idx);
      qlen = __builtin_amdgcn_readlane(ql, idx);
      seq_len = __builtin_amdgcn_readlane(L, idx);
      return true;
    }
    base += total;
  }
  return false;
}

// PRE (taken when the caller asks for no lse): the softmax factor c2 is folded into the Q
// operands, which costs one more bf16 rounding of Q (lse would be off by up to ~5e-3, the
// outputs stay within a bf16 ulp of the unfolded path) and saves the FMA per score.
template <bool FP8, bool PRE>
__global__ __launch_bounds__(kPfWaves * 64, 2) void prefill_kernel(const AttnParams p,
                                                                   const PfTable tab) {
  constexpr int NT = 4;
  constexpr int kElt = FP8 ? 1 : 2;
  // DMA (bf16 cache, folded softmax factor): the K/V tiles go straight from the pages into LDS
  // (global_load_lds_dwordx4: a wave instruction moves 8 token rows x 128 bytes of one KV head),
  // no staging registers, no ds_write; 128-byte rows with permuted segments (see chunk_pipe).
  // Four separate arrays: the compiler can then tell the tile being loaded from the one being
  // read and puts no wait for the loads in front of the reads.
  constexpr bool DMA = PRE && !FP8;
  constexpr int kDmaTile = kChunk * 128;
  __shared__ __align__(16) uint8_t lds_k[2][DMA ? 16 : kPfKTileBytes];  // double-buffered K tile
  __shared__ __align__(16) uint8_t lds_v[2][DMA ? 16 : kPfVTileBytes];  // double-buffered V tile
  __shared__ __align__(1024) uint8_t dma_k0[DMA ? kDmaTile : 16];
  __shared__ __align__(1024) uint8_t dma_k1[DMA ? kDmaTile : 16];
  __shared__ __align__(1024) uint8_t dma_v0[DMA ? kDmaTile : 16];
  __shared__ __align__(1024) uint8_t dma_v1[DMA ? kDmaTile : 16];
  // PRE: every wave's eight Q fragments, in fragment order (see chunk_pipe)
  __shared__ __align__(16) uint8_t lds_q[PRE ? kPfWaves * 8 * kQFragBytes : 16];
  __shared__ int item_lds[8];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int Hkv = p.num_kv_heads;
  const int kvh = blockIdx.x % Hkv;
  // Key-range split (few tiles, long contexts): `KS` consecutive units share one tile and
  // take one part of its key range each.
  const int KS = p.pf_splits;
  const int unit = blockIdx.x / Hkv;
  const int ks_part = KS > 1 ? unit % KS : 0;
  const int tl_slot = blockIdx.x * kPfWaves + wave;
  timeline_start(p, tl_slot);
  const int W = p.window;
  const float c2 = p.softmax_scale * kLog2e * (FP8 ? p.k_scale[kvh] : 1.0f);
  // the lane's rows all belong to one query head: its sink is fetched ahead of its use and
  // parked in LDS (a register held through the chunk loop costs spills)
  __shared__ float lds_sink[kPfWaves * 64];
  lds_sink[tid] = p.sinks ? p.sinks[kvh * kGroup + (i16 & 7)] * kLog2e : -INFINITY;
  int s, tile, row0, qlen, L;
  if (tab.n > 0) {
    // the host listed the tiles: scalar loads alone (lengths still come from the device arrays)
    const int item = KS > 1 ? unit / KS : unit;
    if (item >= tab.n) return;
    const uint32_t e = tab.e[item];
    s = (int)(e & 0xffffu);
    tile = (int)(e >> 16);
    const const_i32_ptr cu = as_constant(p.cu_seqlens_q), sl = as_constant(p.seq_lens);
    row0 = cu[s];
    qlen = cu[s + 1] - row0;
    L = min(sl[s], p.max_blocks_per_seq * kBlock);
    if (qlen < p.qlen_lo || qlen > p.qlen_hi || L < qlen || tile * kPfTok >= qlen) return;
  } else {
    // one wave looks the item up, the others receive it through LDS
    if (wave == 0) {
      int s0 = 0, tile0 = 0, row00 = 0, qlen0 = 0, L0 = 0;
      const bool found = find_prefill_item(p, KS > 1 ? unit / KS : unit, s0, tile0, row00, qlen0, L0);
      if (lane == 0) {
        item_lds[0] = found;
        item_lds[1] = s0;
        item_lds[2] = tile0;
        item_lds[3] = row00;
        item_lds[4] = qlen0;
        item_lds[5] = L0;
      }
    }
    __syncthreads();
    if (!__builtin_amdgcn_readfirstlane(item_lds[0])) return;
    s = __builtin_amdgcn_readfirstlane(item_lds[1]);
    tile = __builtin_amdgcn_readfirstlane(item_lds[2]);
    row0 = __builtin_amdgcn_readfirstlane(item_lds[3]);
    qlen = __builtin_amdgcn_readfirstlane(item_lds[4]);
    L = __builtin_amdgcn_readfirstlane(item_lds[5]);
  }

  const int pos0 = L - qlen;
  const int tq_wg = tile * kPfTok;
  const int pos_first_wg = pos0 + tq_wg;
  const int pos_last_wg = pos0 + min(tq_wg + kPfTok, qlen) - 1;
  int t_begin = (W > 0 ? max(0, pos_first_wg - W + 1) : 0) & ~(kBlock - 1);
  int t_end = pos_last_wg + 1;
  if (KS > 1) {  // this unit's part of the key range, in whole 64-token chunks
    const int per = ((t_end - t_begin + KS - 1) / KS + kChunk - 1) / kChunk * kChunk;
    t_begin += ks_part * per;
    t_end = min(t_end, t_begin + per);  // may leave nothing: empty partials are written
  }
  // this wave's rows
  const int tq0 = tq_wg + wave * kPfWaveTok;
  const bool wave_active = tq0 < qlen;
  const int pos_first = pos0 + tq0;
  const int pos_last = pos0 + min(tq0 + kPfWaveTok, qlen) - 1;
  const int lo_first = W > 0 ? max(0, pos_first - W + 1) : 0;
  const int lo_last = W > 0 ? max(0, pos_last - W + 1) : 0;

  // cooperative loader: thread -> (row of the 64-token chunk, 32-byte segment of the head row)
  // (a wave loads one page of the chunk: its id is wave-uniform and travels in a scalar register)
  const int ld_row = tid >> 2, ld_seg = tid & 3;
  const int ld_page = wave;
  const uint32_t row_bytes = (uint32_t)Hkv * kHeadDim * kElt;
  const size_t page_bytes = (size_t)kBlock * row_bytes;
  const uint32_t gl_off = (uint32_t)(ld_row & 15) * row_bytes + (uint32_t)kvh * (kHeadDim * kElt) +
                          (uint32_t)ld_seg * (16 * kElt);
  const uint32_t st_off_k = (uint32_t)ld_row * kPfKRowBytes + ld_seg * 32;
  const uint32_t st_off_v = (uint32_t)ld_row * kPfVRowBytes + ld_seg * 32;
  const const_i32_ptr bt = as_constant(p.block_table + (size_t)s * p.max_blocks_per_seq);
  const int nblk_total = (t_end + kBlock - 1) / kBlock;

  u32x4 kr[kElt], vr[kElt];
  auto fetch = [&](const int tc) {  // global -> registers for chunk starting at token tc
    const int blk = clamp_page(bt[min(tc / kBlock + ld_page, nblk_total - 1)], p.last_block);
#pragma unroll
    for (int e = 0; e < kElt; ++e) {
      kr[e] = u32x4{0, 0, 0, 0};
      vr[e] = u32x4{0, 0, 0, 0};
    }
    if (tc + ld_page * kBlock < t_end) {
      const uint8_t *kp = p.k_cache + (size_t)blk * page_bytes + gl_off;
      const uint8_t *vp = p.v_cache + (size_t)blk * page_bytes + gl_off;
#pragma unroll
      for (int e = 0; e < kElt; ++e) {
        kr[e] = ldg128(kp + 16 * e);
        vr[e] = ldg128(vp + 16 * e);
      }
    }
  };
  auto stash = [&](const int tc, const int buf) {  // registers -> LDS tile (bf16)
    u32x4 k0, k1, v0, v1;
    if constexpr (FP8) {
      uint32_t a4[4], b4[4];
      fp8x8_to_bf16x8(kr[0][0], kr[0][1], a4);
      fp8x8_to_bf16x8(kr[0][2], kr[0][3], b4);
      k0 = u32x4{a4[0], a4[1], a4[2], a4[3]};
      k1 = u32x4{b4[0], b4[1], b4[2], b4[3]};
      fp8x8_to_bf16x8(vr[0][0], vr[0][1], a4);
      fp8x8_to_bf16x8(vr[0][2], vr[0][3], b4);
      v0 = u32x4{a4[0], a4[1], a4[2], a4[3]};
      v1 = u32x4{b4[0], b4[1], b4[2], b4[3]};
    } else {
      k0 = kr[0];
      k1 = kr[kElt - 1];
      v0 = vr[0];
      v1 = vr[kElt - 1];
    }
    if (tc + ld_row >= L) {  // rows past the sequence end may hold anything: V must be 0
      v0 = u32x4{0, 0, 0, 0};
      v1 = u32x4{0, 0, 0, 0};
    }
    *(u32x4 *)(&lds_k[buf][st_off_k]) = k0;
    *(u32x4 *)(&lds_k[buf][st_off_k + 16]) = k1;
    *(u32x4 *)(&lds_v[buf][st_off_v]) = v0;
    *(u32x4 *)(&lds_v[buf][st_off_v + 16]) = v1;
  };

  // DMA loader: wave w moves the chunk's page w (tile rows 16 w .. 16 w + 15) as two pieces of
  // 8 rows per tensor; lane (r, sl) = (lane / 8, lane % 8) fills slot sl of its row.  Rows past
  // the sequence end repeat its last row (real, finite data; their scores are masked), as the
  // pages behind them may never have been written.
  const int dma_r = lane >> 3, dma_sl = lane & 7;
  auto dma = [&](uint8_t *kbuf, uint8_t *vbuf, const int tc) {
    const int blk = clamp_page(bt[min(tc / kBlock + wave, nblk_total - 1)], p.last_block);
    const uint8_t *kp = p.k_cache + (size_t)blk * page_bytes + (uint32_t)kvh * 128;
    const uint8_t *vp = p.v_cache + (size_t)blk * page_bytes + (uint32_t)kvh * 128;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = 8 * h + dma_r;  // row of the page = tile row - 16 wave
      const int tok = min(tc + 16 * wave + row, L - 1);
      const uint32_t off = (uint32_t)(tok & 15) * row_bytes;
      const int kseg = dma_sl ^ (4 * h + (dma_r >> 1));
      const int vseg = dma_sl ^ ((dma_r >> 1) << 1);
      __builtin_amdgcn_global_load_lds((pf_gptr_t *)(kp + off + kseg * 16),
                                       (pf_lptr_t *)(kbuf + (2 * wave + h) * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((pf_gptr_t *)(vp + off + vseg * 16),
                                       (pf_lptr_t *)(vbuf + (2 * wave + h) * 1024), 16, 0, 0);
    }
  };

  // the first K/V tile is requested before the Q operands: both are in flight together
  timeline_mark(p, tl_slot, 0);
  if (t_begin < t_end) {
    if constexpr (DMA) dma(dma_k0, dma_v0, t_begin);
    else fetch(t_begin);
  }

  Frag8 qf[NT][2];
  RowInfo ri;
  load_q<NT, PRE>(p, row0, qlen, wave_active ? tq0 : tq_wg, kvh, pos0, qf, ri, c2);
  uint8_t *q_lds = &lds_q[0] + (PRE ? wave * (8 * kQFragBytes) + lane * 16 : 0);
  if constexpr (PRE) {  // (wave-private: no barrier, the reads wait for the wave's own stores)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int h = 0; h < 2; ++h) *(u32x4 *)(q_lds + (2 * nt + h) * kQFragBytes) = qf[nt][h].u;
  }
  bool maybe_fresh = true;
  float m[NT];
  f32x4 lacc[NT], acc[NT][4];
  // PRE: the rows' row sums as scalars and the MFMA seeds -(reference) of the four tiles
  float lsum[NT];
  f32x4 zs[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    m[nt] = kNegBig;
    lacc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    lsum[nt] = 0.f;
    zs[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  if constexpr (DMA) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of the first tile is in LDS
    __syncthreads();
    timeline_mark(p, tl_slot, 1);
    const int sw_k = (i16 >> 1) & 7;
    const uint32_t k_off = (uint32_t)i16 * 128 + (uint32_t)((2 * g) ^ sw_k) * 16;
    const int v_row = 4 * g + (i16 >> 2);
    const uint32_t v_off = (uint32_t)v_row * 128 + 8 * (i16 & 3);
    const int v_sw = 32 * ((v_row >> 1) & 3);
    auto iter = [&](uint8_t *kcur, uint8_t *vcur, uint8_t *knxt, uint8_t *vnxt, const int tc) {
      if (tc + kChunk < t_end) dma(knxt, vnxt, tc + kChunk);
      if (wave_active && tc <= pos_last && tc + kChunk > lo_first) {
        const bool need_mask = (tc < lo_last) || (tc + kChunk > pos_first + 1);
        chunk_pipe<128, true>(kcur + k_off, kcur + (k_off ^ 16), kBlock * 128, vcur + v_off, v_sw, q_lds,
                              maybe_fresh, m, zs, lsum, acc, ri, tc, need_mask);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): my share of the next tile has landed
      __syncthreads();
    };
    for (int tc = t_begin; tc < t_end; tc += 2 * kChunk) {
      iter(dma_k0, dma_v0, dma_k1, dma_v1, tc);
      if (tc + kChunk < t_end) iter(dma_k1, dma_v1, dma_k0, dma_v0, tc + kChunk);
    }
  } else {
  if (t_begin < t_end) stash(t_begin, 0);
  __syncthreads();
  timeline_mark(p, tl_slot, 1);
  int cur = 0;
  for (int tc = t_begin; tc < t_end; tc += kChunk, cur ^= 1) {
    const bool has_next = tc + kChunk < t_end;
    if (has_next) fetch(tc + kChunk);
    if (wave_active && tc <= pos_last && tc + kChunk > lo_first) {
      const uint8_t *kt = &lds_k[cur][0] + i16 * kPfKRowBytes + g * 32;
      const uint8_t *v_rd = &lds_v[cur][0] + (4 * g + (i16 >> 2)) * kPfVRowBytes + 8 * (i16 & 3);
      const bool need_mask = (tc < lo_last) || (tc + kChunk > pos_first + 1);
      if constexpr (PRE) {
        chunk_pipe<kPfVRowBytes>(kt, kt + 16, kBlock * kPfKRowBytes, v_rd, 0, q_lds, maybe_fresh, m, zs, lsum,
                                 acc, ri, tc, need_mask);
      } else {
        Frag8 kf[4][2];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          kf[b][0].u = *(const u32x4 *)(kt + b * (kBlock * kPfKRowBytes));
          kf[b][1].u = *(const u32x4 *)(kt + b * (kBlock * kPfKRowBytes) + 16);
        }
        chunk_step<NT, kPfVRowBytes, false>(kf, v_rd, qf, ri, tc, need_mask, c2, m, lacc, acc);
      }
    }
    if (has_next) stash(tc + kChunk, cur ^ 1);
    __syncthreads();
  }
  }
  timeline_mark(p, tl_slot, 2);
  if (!wave_active) return;
  if constexpr (PRE) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) lacc[nt] = f32x4{lsum[nt], lsum[nt], lsum[nt], lsum[nt]};
  }
  if (KS == 1) {
    finish<NT, FP8, false, true>(p, s, kvh, row0, qlen, tq0, true, 0, m, lacc, acc, lds_sink[tid]);
  } else {
    // partials of this part, one cell per (query token, part, head): finish() addresses cells
    // as (s * ws_rows + t), so the sequence's first row with one row per "sequence" gives the
    // token's own index
    AttnParams pp = p;
    pp.ws_ml = p.pf_ml;
    pp.ws_acc = p.pf_acc;
    pp.ws_rows = 1;
    pp.nparts_max = KS;
    finish<NT, FP8>(pp, row0, kvh, row0, qlen, tq0, false, ks_part, m, lacc, acc);
  }
  timeline_end(p, tl_slot, (t_end - t_begin + kChunk - 1) / kChunk);
}

// Merge of the key-range parts of the prefill kernel.  grid = (Hq / 4, num_q_tokens); one wave
// per (query token, head), a lane per head dim.  Tokens of sequences outside the prefill class
// (their rows come from the split-KV kernels) are left alone.
__global__ __launch_bounds__(256) void prefill_merge_kernel(const AttnParams p) {
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int row = blockIdx.y;
  // sequence of this row: last s with cu_seqlens_q[s] <= row
  int lo = 0, hi = p.num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (p.cu_seqlens_q[mid] <= row) lo = mid; else hi = mid - 1;
  }
  const int qlen = p.cu_seqlens_q[lo + 1] - p.cu_seqlens_q[lo];
  if (qlen < p.qlen_lo || qlen > p.qlen_hi || p.seq_lens[lo] < qlen) return;
  const int KS = p.pf_splits, Hq = p.num_q_heads;
  const size_t base = (size_t)row * KS * Hq + head;
  const float sink = p.sinks ? p.sinks[head] : -INFINITY;
  float M = sink;
  for (int j = 0; j < KS; ++j) {
    const float2 ml = *(const float2 *)(p.pf_ml + (base + (size_t)j * Hq) * 2);
    if (ml.y > 0.f) M = fmaxf(M, ml.x);
  }
  float den = fast_exp2((sink - M) * kLog2e), o = 0.f;
  for (int j = 0; j < KS; ++j) {
    const float2 ml = *(const float2 *)(p.pf_ml + (base + (size_t)j * Hq) * 2);
    if (!(ml.y > 0.f)) continue;  // an empty part: its cell may hold anything
    const float w = ml.y * fast_exp2((ml.x - M) * kLog2e);
    den += w;
    o += w * (float)p.pf_acc[(base + (size_t)j * Hq) * kHeadDim + lane];
  }
  // den > 0: a prefill row always sees its own key, so some part is non-empty
  const size_t orow = (size_t)row * Hq + head;
  const float r = o / den;
  const uint32_t mine = __float_as_uint(r), next = __shfl_down(mine, 1);
  if ((lane & 1) == 0)
    *(uint32_t *)(p.out + orow * kHeadDim + lane) = pack_bf16(__uint_as_float(mine), __uint_as_float(next));
  if (p.lse && lane == 0) p.lse[orow] = M + __log2f(den) * kLn2;
}


// ---------------------------------------------------------------------------------------
// Cross-partition merge.  grid = (Hq / 4, num_seqs * ws_rows); one wave per (row, head).
// The (m, l) pairs of up to 64 partitions are fetched one per lane and the weights
// l_c e^(m_c - M) formed lane-parallel.  The partitions' normalised outputs (fp16) are read
// four partitions per load instruction: lane (g, q) = (lane / 16, lane % 16) takes dims
// 4q..4q+3 of partitions g, g+4, g+8, ..., eight loads in flight, and the four lane groups
// are summed at the end.  Sequences finished by the split-KV kernel itself (one partition)
// and sequences outside [qlen_lo, qlen_hi] are skipped.
// ---------------------------------------------------------------------------------------
//
// EAGER (launches of a few rows, where the call is a chain of memory latencies): the (m, l)
// pairs and the first 32 partitions' outputs are requested before the sequence's length, and
// with it the number of partitions that were written, is known; cells beyond that number
// are dropped once it is.
template <bool EAGER>
__global__ __launch_bounds__(256) void lse_merge_kernel(const AttnParams p) {
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int wsrow = blockIdx.y;
  const int s = wsrow / p.ws_rows, t = wsrow % p.ws_rows;
  // Everything that does not depend on another load is requested at once, before the first
  // branch: the row's place in the batch, the sequence's length, the launch's partition slot,
  // the sequence's piece count and the (m, l) pairs of the first 64 cells (cells that were not
  // written hold anything and are dropped once the count is known).  Taken one after the other
  // these were five dependent round trips of a kernel that lasts seven.
  float2 ml_early = make_float2(-INFINITY, 0.f);
  uint2 v_early[8];
  {
    const size_t base = (size_t)wsrow * p.nparts_max * p.num_q_heads + head;
    if (lane < p.nparts_max) ml_early = *(const float2 *)(p.ws_ml + (base + (size_t)lane * p.num_q_heads) * 2);
  }
  const int L_dev = p.seq_lens[s];
  const int P_dev = p.plan_slot ? p.plan_slot[0] : p.partition;
  const int parts_dev = p.nparts_max > 1 ? p.seq_parts[s] : 1;
  int row0 = s, qlen = 1;
  if (p.cu_seqlens_q) {
    row0 = p.cu_seqlens_q[s];
    qlen = p.cu_seqlens_q[s + 1] - row0;
  }
  if (EAGER) {
    const size_t base = (size_t)wsrow * p.nparts_max * p.num_q_heads + head;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = 4 * j + (lane >> 4);
      v_early[j] = make_uint2(0u, 0u);
      if (c < p.nparts_max)
        v_early[j] = *(const uint2 *)(p.ws_acc + (base + (size_t)c * p.num_q_heads) * kHeadDim + (lane & 15) * 4);
    }
  }
  if (qlen < p.qlen_lo || qlen > p.qlen_hi || qlen > p.ws_rows || t >= qlen) return;
  const int L = min(L_dev, p.max_blocks_per_seq * kBlock);  // as the split-KV kernels read it
  if (L < qlen) return;
  // run-time partition: recorded by the split-KV launch of this class; else the caller's
  const int P = P_dev;
  int nparts;
  if (P & kEvenFlag) {  // an even split with pieces of no common size left the count per sequence
    nparts = min(parts_dev, p.nparts_max);
  } else {
    if (P < 64 || (P & 63) != 0) return;  // (a slot no split-KV launch has written: nothing to merge)
    nparts = num_partitions(p, L - kv_begin(L, qlen, p.window), P);
  }
  if (nparts <= 1) return;

  const int g = lane >> 4, q = lane & 15;
  // cell (row, partition c, head) sits at ((row * nparts_max + c) * Hq + head)
  const size_t base = (size_t)wsrow * p.nparts_max * p.num_q_heads + head;
  const size_t cstride = p.num_q_heads;
  const _Float16 *acc_row = p.ws_acc + base * kHeadDim + q * 4;
  const float sink = p.sinks ? p.sinks[head] : -INFINITY;
  // the first 64 partitions' (m, l), kept for both passes
  float2 ml0 = make_float2(-INFINITY, 0.f);
  if (lane < nparts) ml0 = ml_early;
  // pass 1: global maximum over non-empty partitions and the sink
  float M = sink;
  if (ml0.y > 0.f) M = fmaxf(M, ml0.x);
  for (int c = 64 + lane; c < nparts; c += 64) {
    const float2 ml = *(const float2 *)(p.ws_ml + (base + c * cstride) * 2);
    if (ml.y > 0.f) M = fmaxf(M, ml.x);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
  // pass 2: weights per lane, then the weighted sum of the partitions' outputs
  float den = 0.f;
  float o[4] = {0.f, 0.f, 0.f, 0.f};
  for (int c0 = 0; c0 < nparts; c0 += 64) {
    float2 ml = ml0;
    if (c0 > 0) {
      ml = make_float2(-INFINITY, 0.f);
      if (c0 + lane < nparts) ml = *(const float2 *)(p.ws_ml + (base + (c0 + lane) * cstride) * 2);
    }
    const float lw = ml.y > 0.f ? ml.y * fast_exp2((ml.x - M) * kLog2e) : 0.f;
    den += lw;
#pragma unroll
    for (int j0 = 0; j0 < 16; j0 += 8) {
      if (c0 + 4 * j0 >= nparts) break;
      uint2 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int c = c0 + 4 * (j0 + j) + g;
        v[j] = make_uint2(0u, 0u);  // never multiply an unwritten cell, it may hold a NaN
        if (EAGER && c0 == 0 && j0 == 0) {
          if (c < nparts) v[j] = v_early[j];
        } else {
          // (16 lanes take one 128-byte cell: whole lines, read once: streaming hint)
          if (c < nparts) {
            const u32x2 x = __builtin_nontemporal_load((const u32x2 *)(acc_row + (size_t)c * cstride * kHeadDim));
            v[j] = make_uint2(x[0], x[1]);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float w = __shfl(lw, 4 * (j0 + j) + g);
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        const half2_t lo = __builtin_bit_cast(half2_t, v[j].x), hi = __builtin_bit_cast(half2_t, v[j].y);
        o[0] += (float)lo[0] * w;
        o[1] += (float)lo[1] * w;
        o[2] += (float)hi[0] * w;
        o[3] += (float)hi[1] * w;
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) den += __shfl_xor(den, off);
  den += fast_exp2((sink - M) * kLog2e);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o[e] += __shfl_xor(o[e], 16);
    o[e] += __shfl_xor(o[e], 32);
  }
  const size_t orow = (size_t)(row0 + t) * p.num_q_heads + head;
  if (g == 0) {
    const float inv = 1.f / den;
    *(uint2 *)(p.out + orow * kHeadDim + q * 4) =
        make_uint2(pack_bf16(o[0] * inv, o[1] * inv), pack_bf16(o[2] * inv, o[3] * inv));
  }
  if (p.lse && lane == 0) p.lse[orow] = M + __log2f(den) * kLn2;
}

// ---------------------------------------------------------------------------------------
// Slot-mapped KV write.  grid = num_tokens, block = 128: thread e moves 8 elements of the
// token's K row (first Hkv*8 threads) or V row (next Hkv*8 threads).
// ---------------------------------------------------------------------------------------
template <bool FP8>
__global__ __launch_bounds__(128) void kv_write_kernel(const uint16_t *__restrict__ k_new,
                                                       const uint16_t *__restrict__ v_new,
                                                       uint8_t *__restrict__ k_cache,
                                                       uint8_t *__restrict__ v_cache,
                                                       const int64_t *__restrict__ slot_mapping,
                                                       const float *__restrict__ k_scale,
                                                       const float *__restrict__ v_scale,
                                                       const int Hkv, const int64_t num_slots) {
  const int t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= num_slots) return;
  const int per = Hkv * (kHeadDim / 8);  // 16-byte groups per row
  for (int e = threadIdx.x; e < 2 * per; e += blockDim.x) {
    const bool is_v = e >= per;
    const int idx = is_v ? e - per : e;
    const uint16_t *src = (is_v ? v_new : k_new) + ((size_t)t * per + idx) * 8;
    uint8_t *dst_base = is_v ? v_cache : k_cache;
    const u32x4 raw = *(const u32x4 *)src;
    if constexpr (FP8) {
      const float sc = (is_v ? v_scale : k_scale)[idx / (kHeadDim / 8)];
      uint32_t o[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t h = (raw[j >> 1] >> ((j & 1) * 16)) & 0xffffu;
        const float x = __fdiv_rn(bf16_bits_to_f32(h), sc);
        o[j >> 2] |= fp8_e4m3_encode(x) << ((j & 3) * 8);
      }
      *(u32x2 *)(dst_base + ((size_t)slot * per + idx) * 8) = u32x2{o[0], o[1]};
    } else {
      *(u32x4 *)(dst_base + ((size_t)slot * per + idx) * 16) = raw;
    }
  }
}

// ---------------------------------------------------------------------------------------
// Fused rotary embedding + QKV split + slot-mapped KV write: the step in front of the
// attention path.  grid = num_tokens, block = 4 * (Hq + 2 Hkv) threads: a thread takes 8
// dims d..d+7 and their partners d+32.. of one head row (the half-split rotation pairs
// dim i with dim i + 32), so it moves two 16-byte pieces in and two out.
//   o1 = fma(-x2, sin, x1 * cos),  o2 = fma(x1, sin, x2 * cos)      (fp32, one rounding each
//   for the product and the fused step), rounded to bf16 nearest-even; K rows then go into
//   the cache exactly as kv_write_kernel stores a bf16 row (bit copy, or fp8 quantisation
//   of the bf16-rounded value), V rows are moved without rotation.
// ---------------------------------------------------------------------------------------
template <bool FP8>
__global__ __launch_bounds__(1024) void rope_kv_write_kernel(
    const uint16_t *__restrict__ qkv, const int32_t *__restrict__ positions,
    const float *__restrict__ cos_sin, const int max_pos, uint16_t *__restrict__ q_out,
    uint8_t *__restrict__ k_cache, uint8_t *__restrict__ v_cache,
    const int64_t *__restrict__ slot_mapping, const float *__restrict__ k_scale,
    const float *__restrict__ v_scale, const int Hq, const int Hkv, const int64_t num_slots) {
  const int t = blockIdx.x;
  const int head = threadIdx.x >> 2, piece = threadIdx.x & 3;  // head row of [q | k | v]
  const size_t row = (size_t)(Hq + 2 * Hkv) * kHeadDim;
  const uint16_t *src = qkv + (size_t)t * row + (size_t)head * kHeadDim + 8 * piece;
  const u32x4 r1 = *(const u32x4 *)src, r2 = *(const u32x4 *)(src + 32);
  const bool is_v = head >= Hq + Hkv;
  u32x4 o1 = r1, o2 = r2;
  if (!is_v) {
    const int pos = min(max(positions[t], 0), max_pos - 1);  // out-of-range stays in the table
    const float *cs = cos_sin + (size_t)pos * kHeadDim + 8 * piece;
    float c[8], sn[8];
    *(f32x4 *)&c[0] = *(const f32x4 *)cs;
    *(f32x4 *)&c[4] = *(const f32x4 *)(cs + 4);
    *(f32x4 *)&sn[0] = *(const f32x4 *)(cs + 32);
    *(f32x4 *)&sn[4] = *(const f32x4 *)(cs + 36);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a[2], b[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float x1 = bf16_bits_to_f32((r1[j] >> (16 * h)) & 0xffffu);
        const float x2 = bf16_bits_to_f32((r2[j] >> (16 * h)) & 0xffffu);
        const float cc = c[2 * j + h], ss = sn[2 * j + h];
        a[h] = __builtin_fmaf(-x2, ss, __fmul_rn(x1, cc));
        b[h] = __builtin_fmaf(x1, ss, __fmul_rn(x2, cc));
      }
      o1[j] = pack_bf16(a[0], a[1]);
      o2[j] = pack_bf16(b[0], b[1]);
    }
  }
  if (head < Hq) {
    uint16_t *dst = q_out + ((size_t)t * Hq + head) * kHeadDim + 8 * piece;
    *(u32x4 *)dst = o1;
    *(u32x4 *)(dst + 32) = o2;
    return;
  }
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= num_slots) return;
  const int kh = is_v ? head - Hq - Hkv : head - Hq;
  uint8_t *cache = is_v ? v_cache : k_cache;
  const size_t elem = ((size_t)slot * Hkv + kh) * kHeadDim + 8 * piece;
  if constexpr (FP8) {
    const float sc = (is_v ? v_scale : k_scale)[kh];
    u32x2 q1 = {0, 0}, q2 = {0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float x1 = __fdiv_rn(bf16_bits_to_f32((o1[j >> 1] >> ((j & 1) * 16)) & 0xffffu), sc);
      const float x2 = __fdiv_rn(bf16_bits_to_f32((o2[j >> 1] >> ((j & 1) * 16)) & 0xffffu), sc);
      q1[j >> 2] |= fp8_e4m3_encode(x1) << ((j & 3) * 8);
      q2[j >> 2] |= fp8_e4m3_encode(x2) << ((j & 3) * 8);
    }
    *(u32x2 *)(cache + elem) = q1;
    *(u32x2 *)(cache + elem + 32) = q2;
  } else {
    *(u32x4 *)(cache + elem * 2) = o1;
    *(u32x4 *)(cache + (elem + 32) * 2) = o2;
  }
}

// ---------------------------------------------------------------------------------------
// Host-side launchers (called from the C ABI after validation).
// ---------------------------------------------------------------------------------------
// Workgroups of kernel `fn` the whole device holds at once (cached per instantiation),
// from the kernel's own register and LDS footprint: a gfx950 SIMD has 512 VGPRs per lane
// (allocated in eights, at most 8 waves), a CU has 4 SIMDs and 160 KB of LDS.
template <typename F>
static int device_fill(F fn, int block) {
  hipFuncAttributes attr;
  hipDeviceProp_t prop;
  int dev = 0;
  if (hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(fn)) != hipSuccess ||
      hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
    return 512;
  const int regs = max(8, (attr.numRegs + 7) / 8 * 8);
  const int waves_per_simd = max(1, min(8, 512 / regs));
  const int waves_per_wg = block / 64;
  int per_cu = max(1, 4 * waves_per_simd / waves_per_wg);
  if (attr.sharedSizeBytes > 0)
    per_cu = min(per_cu, max(1, (int)(prop.maxSharedMemoryPerMultiProcessor / attr.sharedSizeBytes)));
  if (getenv("EID_DEBUG"))
    fprintf(stderr, "[eid] kernel regs=%d lds=%zu block=%d -> %d workgroups/CU x %d CUs\n",
            attr.numRegs, attr.sharedSizeBytes, block, per_cu, prop.multiProcessorCount);
  return per_cu * max(1, prop.multiProcessorCount);
}

int device_cus() {
  static const int cus = [] {
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
    return max(1, prop.multiProcessorCount);
  }();
  return cus;
}

// Measurement aids, compiled into the measurement build only (-DEID_MEASURE): the serving
// library carries neither the entry points nor their process-wide state.
//  * a device buffer of `entries` records of 64 bytes that the next prefill launches of the
//    process fill with per-wave time stamps (null: off; launches with more waves than entries
//    leave the buffer alone);
//  * a pair of HIP events that the next decode launches attach to the split-KV kernel's own
//    dispatch (hipExtLaunchKernel): the time between them is the kernel's duration as a
//    profiler reports it, without the gaps that events recorded around a launch include.
// The settings are read once per launch (atomics); what they point to is the caller's and
// must outlive the setting.
#ifdef EID_MEASURE
static std::atomic<unsigned long long *> g_timeline{nullptr};
static std::atomic<long long> g_timeline_entries{0};
void set_timeline(void *buf, long long entries) {
  g_timeline_entries.store(0);
  g_timeline.store(static_cast<unsigned long long *>(buf));
  g_timeline_entries.store(buf ? entries : 0);
}
static unsigned long long *timeline_for(const long long waves) {
  return waves <= g_timeline_entries.load() ? g_timeline.load() : nullptr;
}
static std::atomic<hipEvent_t> g_kernel_start{nullptr}, g_kernel_stop{nullptr};
void set_kernel_events(void *start, void *stop) {
  g_kernel_start.store(static_cast<hipEvent_t>(start));
  g_kernel_stop.store(static_cast<hipEvent_t>(stop));
}
//  * a switch for the even split with the caller's partition: 1 = a partial per partition, all
//    merged by the merge kernel; 0 = one partial per piece; -1 = as EID_STORE_EVERY_PARTITION says.
static std::atomic<int> g_store_every_partition{-1};
void set_store_every_partition(int mode) { g_store_every_partition.store(mode); }
int store_every_partition_override() { return g_store_every_partition.load(); }
#else
static unsigned long long *timeline_for(const long long) { return nullptr; }
#endif

// Launches `kern`; in the measurement build, with the two events attached to the dispatch when
// they are set and the launch is one that they are meant for (`timed`).
template <typename K, typename... A>
static hipError_t launch_kernel(K kern, dim3 grid, dim3 block, unsigned shmem, hipStream_t st,
                                bool timed, const A &...a) {
#ifdef EID_MEASURE
  const hipEvent_t e0 = g_kernel_start.load(), e1 = g_kernel_stop.load();
  if (timed && e0 && e1) {
    void *kargs[] = {const_cast<void *>(static_cast<const void *>(&a))...};
    return hipExtLaunchKernel(reinterpret_cast<const void *>(kern), grid, block, kargs, shmem, st, e0, e1, 0);
  }
#else
  (void)timed;
#endif
  kern<<<grid, block, shmem, st>>>(a...);
  return hipGetLastError();
}

template <int NT, bool FP8, int WAVES, int RS = 1, bool PAIR = false, bool DMA = false>
static int fill_of() {
  static const int fill = device_fill(splitkv_kernel<NT, FP8, WAVES, RS, PAIR, DMA>, WAVES * 64);
  return fill;
}

template <int NT, bool FP8, bool DMA = false>
static int fill_t(int waves) {
  switch (waves) {
    case 8: return fill_of<NT, FP8, 8, 1, false, DMA>();
    case 4: return fill_of<NT, FP8, 4, 1, false, DMA>();
    case 2: return fill_of<NT, FP8, 2, 1, false, DMA>();
    default: return fill_of<NT, FP8, 1, 1, false, DMA>();
  }
}

static int waves_for(int Hkv) { return Hkv >= 8 ? 8 : Hkv; }

// Workgroups of the split-KV instantiation (ntiles, fp8, Hkv) the device holds at once.
int splitkv_fill(int ntiles, bool fp8, int Hkv, bool pair, bool dma) {
  if (pair && fp8 && ntiles == 1) return fill_of<1, true, 4, 1, true>();  // two KV heads per wave
  const int waves = waves_for(Hkv);
  if (dma && !fp8 && ntiles < 8)
    return ntiles == 1 ? fill_t<1, false, true>(waves) : ntiles == 3 ? fill_t<3, false, true>(waves) : fill_t<4, false, true>(waves);
  if (ntiles == 8) return fp8 ? fill_of<4, true, 8, 2>() : fill_of<4, false, 8, 2>();  // two row groups
  if (ntiles == 16) return fp8 ? fill_of<4, true, 8, 4>() : fill_of<4, false, 8, 4>();  // four
  if (fp8) return ntiles == 1 ? fill_t<1, true>(waves) : ntiles == 3 ? fill_t<3, true>(waves) : fill_t<4, true>(waves);
  return ntiles == 1 ? fill_t<1, false>(waves) : ntiles == 3 ? fill_t<3, false>(waves) : fill_t<4, false>(waves);
}

// Upper bound on the number of work items of a launch, from what the host knows.  Items
// never exceed num_seqs * nparts_max.  With the run-time partition they are at most Tlo
// (one workgroup per CU) or T (one device fill) in the single-fill tiers, and
// sum/P3 + num_seqs in the multi-fill regime, where P3 = min(cap, max(floor, ~sum/(3T)))
// makes sum/P3 <= min(sum/floor, max(sum/cap, 3T)).  Without the caller's sum_kv_len the
// sum is bounded by num_seqs * max_kv_len.  With it, the host can often tell which tier the
// kernels will take: their first estimate ceil64(total / (Tx - active)) grows with total
// and with active, so if it is below the cap for (sum_kv_len, num_seqs) it is below the cap
// for the real batch, and the tier Tx is taken.
static long long item_bound(const AttnParams &p) {
  if (p.exact_items > 0) return p.exact_items;
  const long long S = p.num_seqs, T = p.target_items, Tlo = p.target_items_lo;
  if (p.nparts_max == 1) return S;  // workgroup w serves sequence w
  long long items = S * p.nparts_max;
  if (p.dynamic_partition) {
    const long long at_floor =
        S * (((long long)p.nparts_max * p.partition + kDynPartitionFloor - 1) / kDynPartitionFloor + 1);
    items = min(items, max(T, at_floor));
    if (p.sum_kv_len > 0) {
      const long long sum = p.sum_kv_len;
      auto takes_tier = [&](const long long Tx) {
        return S < Tx && ((sum + (Tx - S) - 1) / (Tx - S) + 63) / 64 * 64 < kDynPartitionCap;
      };
      // (the equal-pieces rule for nearly uniform batches never goes below half the cap)
      const long long multi =
          min(sum / kDynPartitionFloor, max(2 * sum / kDynPartitionCap, 3 * T)) + S + 16;
      if (Tlo < T && takes_tier(Tlo)) items = min(items, Tlo);
      else if (takes_tier(T)) items = min(items, T);
      else items = min(items, max(T, multi));
    }
  } else if (p.sum_kv_len > 0) {
    items = min(items, p.sum_kv_len / p.partition + S);
  }
  return items;
}

template <int NT, bool FP8, int WAVES, int RS = 1, bool PAIR = false>
static hipError_t launch_splitkv_w(const AttnParams &p, hipStream_t st) {
  dim3 grid((unsigned)item_bound(p), p.num_kv_heads / (WAVES / RS) / (PAIR ? 2 : 1));
  if constexpr (!FP8 && RS == 1) {
    if (p.dma)  // (never beside a prefill launch: its LDS leaves no room for one)
      return launch_kernel(splitkv_kernel<NT, FP8, WAVES, RS, PAIR, true>, grid, dim3(WAVES * 64), 0, st, true, p);
  }
  // With a prefill launch beside it (mixed batch, p.share_cus): one 8-wave workgroup per CU.
  // A second resident workgroup adds little to a kernel that streams from HBM (it only
  // covers the prologues of many short items), while half of the CU's registers left free
  // let a prefill workgroup run next to it.  The cap is a request for unused dynamic LDS: two
  // such workgroups no longer fit a CU's 160 KB, one plus a prefill workgroup does.
  const int kPad = (WAVES == 8 && p.share_cus) ? 16384 : 0;
  if (kPad > 0) {  // once per device: allow the kernel its dynamic LDS on top of the static tile
    static std::atomic<bool> allowed[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {
      e = hipFuncSetAttribute((const void *)splitkv_kernel<NT, FP8, WAVES, RS, PAIR>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, kPad);
      if (e != hipSuccess) return e;
      if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);
    }
  }
  return launch_kernel(splitkv_kernel<NT, FP8, WAVES, RS, PAIR>, grid, dim3(WAVES * 64), kPad, st, true, p);
}

template <int NT, bool FP8>
static hipError_t launch_splitkv_t(const AttnParams &p, hipStream_t st) {
  switch (waves_for(p.num_kv_heads)) {
    case 8: return launch_splitkv_w<NT, FP8, 8>(p, st);
    case 4: return launch_splitkv_w<NT, FP8, 4>(p, st);
    case 2: return launch_splitkv_w<NT, FP8, 2>(p, st);
    default: return launch_splitkv_w<NT, FP8, 1>(p, st);
  }
}

// Item count of the one-workgroup-per-CU tier of the run-time partition rule.
static int fill_lo(int target_items) { return min(target_items, device_cus()); }

// Upper bound on the (sequence, partition) pairs of a short-span launch: the host knows the
// longest span, and perhaps the sum of the lengths (which bounds the spans without a window).
long long shortspan_items(int num_seqs, int nparts_max, long long sum_kv_len, int window) {
  long long items = (long long)num_seqs * nparts_max;
  if (nparts_max > 1 && sum_kv_len > 0 && window == 0)
    items = min(items, sum_kv_len / kShortSpanMax + num_seqs);
  return items;
}

// Short-span launch: see shortspan_kernel.  The caller has checked that no sequence spans
// more than kShortSpanMax tokens.
hipError_t launch_shortspan(const AttnParams &p, int ntiles, bool fp8, hipStream_t st,
                            const ItemTable *tab) {
  if (tab && ntiles == 1 && p.nparts_max > 1) {  // decode launch with the host's item list
    dim3 grid((unsigned)tab->n, p.num_kv_heads);
    if (fp8) shortspan_table_kernel<1, true><<<grid, kShortWaves * 64, 0, st>>>(p, *tab);
    else shortspan_table_kernel<1, false><<<grid, kShortWaves * 64, 0, st>>>(p, *tab);
    return hipGetLastError();
  }
  const long long items = p.exact_items > 0 && p.nparts_max > 1
                              ? p.exact_items
                              : shortspan_items(p.num_seqs, p.nparts_max, p.sum_kv_len, p.window);
  dim3 grid((unsigned)items, p.num_kv_heads);
  if (fp8) {
    if (ntiles == 1) shortspan_kernel<1, true><<<grid, kShortWaves * 64, 0, st>>>(p);
    else if (ntiles == 3) shortspan_kernel<3, true><<<grid, kShortWaves * 64, 0, st>>>(p);
    else shortspan_kernel<4, true><<<grid, kShortWaves * 64, 0, st>>>(p);
  } else {
    if (ntiles == 1) shortspan_kernel<1, false><<<grid, kShortWaves * 64, 0, st>>>(p);
    else if (ntiles == 3) shortspan_kernel<3, false><<<grid, kShortWaves * 64, 0, st>>>(p);
    else shortspan_kernel<4, false><<<grid, kShortWaves * 64, 0, st>>>(p);
  }
  return hipGetLastError();
}
// Whether the short-span kernel should serve a launch of `num_items` (sequence, 512-key
// partition) pairs: no more workgroups (one per item and KV head) than the device holds at
// once; beyond that the split-KV kernel's one workgroup per item with longer partitions makes
// fewer, better filled rounds.
bool shortspan_applies(int ntiles, bool fp8, long long num_items, int Hkv) {
  if (ntiles >= 8) return false;  // several row groups per KV head: split-KV kernel only
  static const int fill[3][2] = {
      {device_fill(shortspan_kernel<1, false>, kShortWaves * 64),
       device_fill(shortspan_kernel<1, true>, kShortWaves * 64)},
      {device_fill(shortspan_kernel<3, false>, kShortWaves * 64),
       device_fill(shortspan_kernel<3, true>, kShortWaves * 64)},
      {device_fill(shortspan_kernel<4, false>, kShortWaves * 64),
       device_fill(shortspan_kernel<4, true>, kShortWaves * 64)}};
  return num_items * Hkv <= fill[ntiles == 1 ? 0 : ntiles == 3 ? 1 : 2][fp8 ? 1 : 0];
}

// Workgroups of an even split: resident all at once, one 8-wave workgroup per CU (eight waves
// keep a CU's share of the memory system busy; of two resident workgroups the younger mostly
// waits), smaller workgroups so that a CU holds eight waves (the four-wave head-pair kernel
// of config 4 with one iteration's loads under way per wave: one per CU 294 us, two 267,
// three 271, four 280: more ranges are more pieces to store and merge).  The head-pair kernel
// that keeps two iterations under way per wave is fed by one workgroup per CU (config 4:
// 251 - 253 us against 255 - 256 with two).  EID_EVEN_WGS_PER_CU overrides the number per CU
// for measurements.
template <int NT, bool FP8, int WAVES, bool PAIR = false, bool DMA = false>
static int even_fill_of() {
  static const int fill = device_fill(splitkv_even_kernel<NT, FP8, WAVES, PAIR, DMA>, WAVES * 64);
  return fill;
}
template <int NT, bool FP8, bool DMA = false>
static int even_fill_t(int waves) {
  switch (waves) {
    case 8: return even_fill_of<NT, FP8, 8, false, DMA>();
    case 4: return even_fill_of<NT, FP8, 4, false, DMA>();
    case 2: return even_fill_of<NT, FP8, 2, false, DMA>();
    default: return even_fill_of<NT, FP8, 1, false, DMA>();
  }
}
int even_wgs(int ntiles, bool fp8, int Hkv, bool pair, bool dma, bool all_cus) {
  static const int per_cu_env = [] {
    const char *e = getenv("EID_EVEN_WGS_PER_CU");
    return e ? atoi(e) : 0;
  }();
  int fill, waves;
  bool pair_dma = false;
  if (pair && fp8 && ntiles == 1) {
    pair_dma = dma;
    fill = pair_dma ? even_fill_of<1, true, 4, true, true>() : even_fill_of<1, true, 4, true>();
    waves = 4;
  } else {
    waves = waves_for(Hkv);
    if (fp8) fill = ntiles == 1 ? even_fill_t<1, true>(waves) : ntiles == 3 ? even_fill_t<3, true>(waves) : even_fill_t<4, true>(waves);
    else if (dma) fill = ntiles == 1 ? even_fill_t<1, false, true>(waves) : ntiles == 3 ? even_fill_t<3, false, true>(waves) : even_fill_t<4, false, true>(waves);
    else fill = ntiles == 1 ? even_fill_t<1, false>(waves) : ntiles == 3 ? even_fill_t<3, false>(waves) : even_fill_t<4, false>(waves);
  }
  const int per_cu = per_cu_env > 0 ? per_cu_env : pair_dma ? 1 : max(1, 8 / waves);
  // the streaming kernels saturate the memory system from seven eighths of the CUs, and fewer
  // ranges are fewer pieces: 224 workgroups against 256 on one box, call level: config 2 81.0
  // against 82.0 us, config 3's decode rows 157.8 / 160.8, config 5 1,342 / 1,348, config 4
  // (fp8) 250.0 / 251.6 (192: 80.9, 158.1, 1,341, 261)
  // (all_cus: a partial per partition of the caller's is stored, 346 MB of them on config 5: the
  // stores want every CU, 1,742 us against 1,780)
  const int cus = (dma && !all_cus && per_cu_env <= 0) ? device_cus() * 7 / 8 : device_cus();
  return max(1, min(fill, per_cu * cus) / (Hkv > 8 ? Hkv / 8 : 1));
}

template <int NT, bool FP8, int WAVES, bool PAIR = false>
static hipError_t launch_even_w(const AttnParams &p, const EvenTable &tab, hipStream_t st) {
  dim3 grid((unsigned)(tab.n > 0 ? tab.n : p.even_wgs), p.num_kv_heads / WAVES / (PAIR ? 2 : 1));
  const bool timed = true;
  if constexpr (!FP8) {
    if (p.dma)
      return launch_kernel(splitkv_even_kernel<NT, FP8, WAVES, PAIR, true>, grid, dim3(WAVES * 64), 0, st, timed, p, tab);
  }
  if constexpr (PAIR) {
    if (p.dma_pair)
      return launch_kernel(splitkv_even_kernel<NT, FP8, WAVES, true, true>, grid, dim3(WAVES * 64), 0, st, timed, p, tab);
  }
  if constexpr (FP8 && !PAIR && NT >= 3 && WAVES == 8) {
    if (p.dma_fp8)
      return launch_kernel(splitkv_even_kernel<NT, true, 8, false, true>, grid, dim3(512), 0, st, timed, p, tab);
  }
  // (p.share_cus: one 8-wave workgroup per CU by a request for unused dynamic LDS, see launch_splitkv_w)
  const int kPad = (WAVES == 8 && p.share_cus) ? 16384 : 0;
  if (kPad > 0) {
    static std::atomic<bool> allowed[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {
      e = hipFuncSetAttribute((const void *)splitkv_even_kernel<NT, FP8, WAVES, PAIR>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, kPad);
      if (e != hipSuccess) return e;
      if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);
    }
  }
  return launch_kernel(splitkv_even_kernel<NT, FP8, WAVES, PAIR>, grid, dim3(WAVES * 64), kPad, st, timed, p, tab);
}
template <int NT, bool FP8>
static hipError_t launch_even_t(const AttnParams &p, const EvenTable &tab, hipStream_t st) {
  switch (waves_for(p.num_kv_heads)) {
    case 8: return launch_even_w<NT, FP8, 8>(p, tab, st);
    case 4: return launch_even_w<NT, FP8, 4>(p, tab, st);
    case 2: return launch_even_w<NT, FP8, 2>(p, tab, st);
    default: return launch_even_w<NT, FP8, 1>(p, tab, st);
  }
}
// Even split (see splitkv_even_kernel); `tab` may be null (starts found on the device).
hipError_t launch_even(AttnParams &p, int ntiles, bool fp8, int32_t *plan_slot, hipStream_t st,
                       const EvenTable *tab) {
  static const EvenTable none{};
  const EvenTable &t = tab ? *tab : none;
  p.plan = nullptr;
  p.plan_slot = plan_slot;
  if (fp8) {
    if (ntiles == 1 && p.fp8_pair) return launch_even_w<1, true, 4, true>(p, t, st);
    if (ntiles == 1) return launch_even_t<1, true>(p, t, st);
    if (ntiles == 3) return launch_even_t<3, true>(p, t, st);
    return launch_even_t<4, true>(p, t, st);
  }
  if (ntiles == 1) return launch_even_t<1, false>(p, t, st);
  if (ntiles == 3) return launch_even_t<3, false>(p, t, st);
  return launch_even_t<4, false>(p, t, st);
}

// p.target_items must hold splitkv_fill(ntiles, fp8, Hkv).  On return p.plan is set when a
// plan kernel was run for this launch; the merge launch that follows is given the same
// params so that it uses the same partition.
hipError_t launch_splitkv(AttnParams &p, int ntiles, bool fp8, int32_t *plan_slot, hipStream_t st,
                          const ItemTable *tab) {
  p.target_items_lo = fill_lo(p.target_items);
  p.plan = nullptr;
  p.plan_slot = plan_slot;
  // decode launch with the host's item list (fixed partition, eight KV heads per workgroup)
  if (tab && ntiles == 1 && p.nparts_max > 1 && !p.dynamic_partition && !p.share_cus &&
      waves_for(p.num_kv_heads) == 8) {
    dim3 grid((unsigned)tab->n, p.num_kv_heads / 8);
    if (fp8 && p.fp8_pair) return launch_kernel(splitkv_table_kernel<1, true, 4, true>, grid, dim3(256), 0, st, true, p, *tab);
    if (fp8) return launch_kernel(splitkv_table_kernel<1, true, 8>, grid, dim3(512), 0, st, true, p, *tab);
    if (p.dma) return launch_kernel(splitkv_table_kernel<1, false, 8, false, true>, grid, dim3(512), 0, st, true, p, *tab);
    return launch_kernel(splitkv_table_kernel<1, false, 8>, grid, dim3(512), 0, st, true, p, *tab);
  }
  if (p.nparts_max > 1 && p.exact_items == 0 && item_bound(p) > 4LL * p.target_items) {
    AttnParams q = p;
    plan_kernel<<<1, 64, 0, st>>>(q, plan_slot);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    p.plan = plan_slot;
  }
  if (ntiles == 16)  // 17..32 rows: four waves per KV head
    return fp8 ? launch_splitkv_w<4, true, 8, 4>(p, st) : launch_splitkv_w<4, false, 8, 4>(p, st);
  if (ntiles == 8)  // 9..16 rows: two waves per KV head (the host checked num_kv_heads % 8 == 0)
    return fp8 ? launch_splitkv_w<4, true, 8, 2>(p, st) : launch_splitkv_w<4, false, 8, 2>(p, st);
  if (fp8) {
    // decode rows only, eight KV heads: four waves per workgroup, two KV heads per wave
    if (ntiles == 1 && p.fp8_pair) return launch_splitkv_w<1, true, 4, 1, true>(p, st);
    if (ntiles == 1) return launch_splitkv_t<1, true>(p, st);
    if (ntiles == 3) return launch_splitkv_t<3, true>(p, st);
    return launch_splitkv_t<4, true>(p, st);
  }
  if (ntiles == 1) return launch_splitkv_t<1, false>(p, st);
  if (ntiles == 3) return launch_splitkv_t<3, false>(p, st);
  return launch_splitkv_t<4, false>(p, st);
}

// Upper bound on the prefill kernel's 32-token query tiles: every sequence rounds up by at most
// one tile.
long long prefill_tiles_bound(int num_q_tokens, int num_seqs) {
  return (long long)num_q_tokens / kPfTok + num_seqs;
}

// Lists the query tiles of the launch's class from the host's copies of the lengths, most key
// chunks first (ties in sequence order, later tiles first).  False (tab->n = 0) when the list
// does not fit or an index does not fit its field: the kernel then scans on the device.
bool build_prefill_table(const AttnParams &p, const int32_t *seq_lens_host,
                         const int32_t *cu_seqlens_q_host, PfTable *tab) {
  tab->n = 0;
  if (p.num_seqs > 0xffff) return false;
  struct Item { int32_t chunks; uint32_t e; };
  Item items[kPfTableMax];
  int n = 0;
  for (int s = 0; s < p.num_seqs; ++s) {
    const int qlen = cu_seqlens_q_host[s + 1] - cu_seqlens_q_host[s];
    const int L = (int)std::min<long long>(seq_lens_host[s], (long long)p.max_blocks_per_seq * kBlock);
    if (qlen < p.qlen_lo || qlen > p.qlen_hi || L < qlen) continue;
    const int tiles = (qlen + kPfTok - 1) / kPfTok;
    if (tiles > 0xffff || n + tiles > kPfTableMax) return false;
    const int pos0 = L - qlen;
    for (int t = tiles - 1; t >= 0; --t) {
      const int first = pos0 + t * kPfTok, last = pos0 + std::min((t + 1) * kPfTok, qlen) - 1;
      const int begin = (p.window > 0 ? std::max(0, first - p.window + 1) : 0) & ~(kBlock - 1);
      items[n].chunks = (last + 1 - begin + kChunk - 1) / kChunk;
      items[n].e = (uint32_t)s | (uint32_t)t << 16;
      ++n;
    }
  }
  std::stable_sort(items, items + n, [](const Item &a, const Item &b) { return a.chunks > b.chunks; });
  for (int i = 0; i < n; ++i) tab->e[i] = items[i].e;
  tab->n = n;
  return n > 0;
}

hipError_t launch_prefill(const AttnParams &p, int num_q_tokens, bool fp8, hipStream_t st,
                          const PfTable *tab) {
  static const PfTable none{};  // n == 0: items found on the device
  const bool listed = tab && tab->n > 0;
  const long long items = (listed ? tab->n : prefill_tiles_bound(num_q_tokens, p.num_seqs)) *
                          (long long)max(1, p.pf_splits);
  dim3 grid((unsigned)(items * p.num_kv_heads));
  const PfTable &t = listed ? *tab : none;
  const bool pre = p.lse == nullptr;  // an exact lse needs the unfolded softmax factor
  AttnParams q = p;
  q.timeline = timeline_for((long long)grid.x * kPfWaves);
  const dim3 block(kPfWaves * 64);
  hipError_t e;
  if (fp8) e = pre ? launch_kernel(prefill_kernel<true, true>, grid, block, 0, st, true, q, t)
                   : launch_kernel(prefill_kernel<true, false>, grid, block, 0, st, true, q, t);
  else e = pre ? launch_kernel(prefill_kernel<false, true>, grid, block, 0, st, true, q, t)
               : launch_kernel(prefill_kernel<false, false>, grid, block, 0, st, true, q, t);
  if (e != hipSuccess || p.pf_splits <= 1) return e;
  dim3 mgrid(p.num_q_heads / 4, num_q_tokens);
  prefill_merge_kernel<<<mgrid, 256, 0, st>>>(p);
  return hipGetLastError();
}

constexpr int kMergeEagerCells = 256;  // per head: 2 MiB of reads at most
hipError_t launch_merge(const AttnParams &p, hipStream_t st) {
  dim3 grid(p.num_q_heads / 4, p.num_seqs * p.ws_rows);
  // speculating on cells that may not have been written is cheap for a few rows only
  if ((long long)p.num_seqs * p.ws_rows * min(p.nparts_max, 32) <= kMergeEagerCells)
    lse_merge_kernel<true><<<grid, 256, 0, st>>>(p);
  else
    lse_merge_kernel<false><<<grid, 256, 0, st>>>(p);
  return hipGetLastError();
}

hipError_t launch_rope_kv_write(const uint16_t *qkv, const int32_t *positions,
                                const float *cos_sin, int max_pos, uint16_t *q_out,
                                uint8_t *k_cache, uint8_t *v_cache, const int64_t *slot_mapping,
                                const float *k_scale, const float *v_scale, int Hq, int Hkv,
                                int64_t num_slots, int num_tokens, bool fp8, hipStream_t st) {
  if (num_tokens == 0) return hipSuccess;
  const int block = 4 * (Hq + 2 * Hkv);
  if (fp8)
    rope_kv_write_kernel<true><<<num_tokens, block, 0, st>>>(qkv, positions, cos_sin, max_pos,
                                                            q_out, k_cache, v_cache, slot_mapping,
                                                            k_scale, v_scale, Hq, Hkv, num_slots);
  else
    rope_kv_write_kernel<false><<<num_tokens, block, 0, st>>>(qkv, positions, cos_sin, max_pos,
                                                             q_out, k_cache, v_cache, slot_mapping,
                                                             k_scale, v_scale, Hq, Hkv, num_slots);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------
// Split-KV workspace owned by the library, for the decode entry point that allocates nothing:
// a file-scope device array, one copy per GPU the library runs on, held until the process
// ends.  Its name is a host-side stand-in here, not a device address: host code asks the
// runtime for the address once per device (with that device current) and from then on only
// ever uses that pointer, for kernel arguments as for anything else.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

hipError_t static_scratch(uint8_t **ptr) {
  constexpr int kMaxDevices = 64;
  static std::atomic<uint8_t *> addr[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  uint8_t *p = addr[dev].load(std::memory_order_acquire);
  if (!p) {  // first call on this device (threads racing here obtain the same address)
    void *sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!sym) return hipErrorInvalidSymbol;
    p = static_cast<uint8_t *>(sym);
    addr[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return hipSuccess;
}

hipError_t launch_kv_write(const uint16_t *k_new, const uint16_t *v_new, uint8_t *k_cache,
                           uint8_t *v_cache, const int64_t *slot_mapping, const float *k_scale,
                           const float *v_scale, int Hkv, int64_t num_slots, int num_tokens,
                           bool fp8, hipStream_t st) {
  if (num_tokens == 0) return hipSuccess;
  if (fp8)
    kv_write_kernel<true><<<num_tokens, 128, 0, st>>>(k_new, v_new, k_cache, v_cache,
                                                      slot_mapping, k_scale, v_scale, Hkv,
                                                      num_slots);
  else
    kv_write_kernel<false><<<num_tokens, 128, 0, st>>>(k_new, v_new, k_cache, v_cache,
                                                       slot_mapping, k_scale, v_scale, Hkv,
                                                       num_slots);
  return hipGetLastError();
}

}  // namespace eid
