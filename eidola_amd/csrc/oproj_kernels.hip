// Output projection, the step right after the attention path:
//
//   out[t, n] = bf16( sum_k a[t, k] * w[n, k]  + bias[n] + residual[t, n] )       (fp32 sums)
//
// `a` is the attention output exactly as eid_attn_decode / eid_attn_varlen leave it
// ([num_q_tokens, Hq, 64] bf16 = row-major [T, K] with k = head * 64 + dim), `w` is the
// projection weight in the usual out_features x in_features order ([N, K] bf16, K
// contiguous).  Both MFMA operands are therefore K-contiguous and 16-byte fragments load
// straight from memory with no transposition: the attention kernels do not need a
// head-major output variant.
//
// MFMA roles (v_mfma_f32_16x16x32_bf16): weight rows (features) ride the M dimension, tokens
// the N dimension, so lane (i16, g) = (lane % 16, lane / 16) of a result tile holds features
// 4g..4g+3 of token i16: four consecutive bf16 of an output row, one 8-byte store.
//
// Three kernels:
//   oproj_skinny_kernel  T <= 64 (decode batches).  HBM-bound: the weight (N*K*2 bytes) is
//                        streamed once.  One workgroup per 16 features (per 32 when that
//                        keeps the workgroups within one per CU); its 8 waves deal the
//                        K dimension in 64-element chunks, each wave keeps a whole batch of
//                        weight loads in flight, the partial sums meet in LDS.
//   oproj_tiled_kernel   any T.  128 x 128 (or, for batches too small to fill the device
//                        with that, 64 x 64) tokens x features per workgroup, K in steps of
//                        64 through double-buffered, row-padded LDS tiles.
//   oproj_wide_kernel    T above ~1,000.  K in steps of 64 through two LDS stages filled by
//                        direct global -> LDS loads; 128 x 128 tokens x features per workgroup
//                        of 4 waves, two workgroups per CU, or (when that fills whole rounds of
//                        the device better) 256 x 192 per workgroup of 8 waves, one per CU.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <type_traits>

#include "eid_device.h"
#include "eid_params.h"

namespace eid {

namespace {

__device__ __forceinline__ u32x4 ld16(const uint16_t *p) { return *(const u32x4 *)p; }

// bias + residual + bf16 rounding + 8-byte store of one lane's four features of one token
__device__ __forceinline__ void oproj_store(const f32x4 acc, const uint16_t *bias,
                                            const uint16_t *resid, uint16_t *out,
                                            const size_t row_off, const int n) {
  float v[4] = {acc[0], acc[1], acc[2], acc[3]};
  if (bias) {
    const u32x2 b = *(const u32x2 *)(bias + n);
    v[0] += bf16_bits_to_f32(b[0] & 0xffffu);
    v[1] += bf16_bits_to_f32(b[0] >> 16);
    v[2] += bf16_bits_to_f32(b[1] & 0xffffu);
    v[3] += bf16_bits_to_f32(b[1] >> 16);
  }
  if (resid) {
    const u32x2 r = *(const u32x2 *)(resid + row_off + n);
    v[0] += bf16_bits_to_f32(r[0] & 0xffffu);
    v[1] += bf16_bits_to_f32(r[0] >> 16);
    v[2] += bf16_bits_to_f32(r[1] & 0xffffu);
    v[3] += bf16_bits_to_f32(r[1] >> 16);
  }
  u32x2 o;
  o[0] = pack_bf16(v[0], v[1]);
  o[1] = pack_bf16(v[2], v[3]);
  *(u32x2 *)(out + row_off + n) = o;
}

// Epilogue of the tiled kernels: acc[ft][tt] holds features n_lane + 16 ft .. + 3 of token
// t_lane + 16 tt.  The bias of this lane's features once, then token tile by token tile all
// residual loads of the tile at once (clamped addresses, so that no load sits under a lane's
// branch and none waits for the one before), bf16 rounding, 8-byte stores.
template <int WF, int WT>
__device__ __forceinline__ void oproj_epilogue(const f32x4 (&acc)[WF][WT], const uint16_t *bias,
                                               const uint16_t *resid, uint16_t *out, const int T,
                                               const int N, const int t_lane, const int n_lane) {
  float bv[WF][4];
#pragma unroll
  for (int ft = 0; ft < WF; ++ft) {
    u32x2 b = {0u, 0u};
    if (bias) b = *(const u32x2 *)(bias + min(n_lane + 16 * ft, N - 4));
    bv[ft][0] = bf16_bits_to_f32(b[0] & 0xffffu);
    bv[ft][1] = bf16_bits_to_f32(b[0] >> 16);
    bv[ft][2] = bf16_bits_to_f32(b[1] & 0xffffu);
    bv[ft][3] = bf16_bits_to_f32(b[1] >> 16);
  }
#pragma unroll
  for (int tt = 0; tt < WT; ++tt) {
    const int t = t_lane + 16 * tt;
    const size_t row_off = (size_t)min(t, T - 1) * N;
    u32x2 rv[WF];
#pragma unroll
    for (int ft = 0; ft < WF; ++ft) rv[ft] = u32x2{0u, 0u};
    if (resid) {
#pragma unroll
      for (int ft = 0; ft < WF; ++ft) rv[ft] = *(const u32x2 *)(resid + row_off + min(n_lane + 16 * ft, N - 4));
    }
#pragma unroll
    for (int ft = 0; ft < WF; ++ft) {
      const f32x4 c = acc[ft][tt];
      u32x2 o;
      o[0] = pack_bf16(c[0] + bv[ft][0] + bf16_bits_to_f32(rv[ft][0] & 0xffffu),
                       c[1] + bv[ft][1] + bf16_bits_to_f32(rv[ft][0] >> 16));
      o[1] = pack_bf16(c[2] + bv[ft][2] + bf16_bits_to_f32(rv[ft][1] & 0xffffu),
                       c[3] + bv[ft][3] + bf16_bits_to_f32(rv[ft][1] >> 16));
      if (t < T && n_lane + 16 * ft < N) *(u32x2 *)(out + row_off + n_lane + 16 * ft) = o;
    }
  }
}

constexpr int kSkWaves = 8;
constexpr int kSkChunk = 64;                       // K elements per chunk: one 128-byte line per row
constexpr int kSkSlab = kSkWaves * kSkChunk;       // K elements per round: one chunk per wave
constexpr int kSkRounds = 8;                       // rounds whose weight loads are issued at once
constexpr int kSkRowBytes = kSkSlab * 2 + 16;      // LDS row of an activation slab, padded

}  // namespace

// ---------------------------------------------------------------------------------------
// Streaming kernel.  grid = N / (16 FT), block = 512.  TT = number of 16-token tiles (T <= 16 TT).
// K is walked in rounds of 512 elements; in round r wave w owns chunk 8 r + w.
//   weights      each wave loads the fragments of its chunks of 8 rounds (all of K = 4096)
//                back to back, straight from memory: 16 KiB in flight per wave
//   activations  every workgroup needs all of a[T, K].  Loading its MFMA fragments straight
//                from memory (16 rows x 64 bytes per instruction, rows 2 K bytes apart) runs
//                at a fraction of the cache bandwidth, so a slab of a round (16 TT rows x
//                1 KiB) is fetched with whole-row loads (one row per wave instruction), kept
//                two rounds ahead in registers, passed through a double-buffered LDS tile
//                and read from there as fragments.
// The eight K shares meet in LDS (reusing the slab tiles).  Requires K % 64 == 0.
// ---------------------------------------------------------------------------------------
// FT = 16-feature tiles per workgroup.  A workgroup's cost is mostly its pass over the
// activations, whatever the number of features, and with three or four token tiles only one
// workgroup fits a CU (LDS): when N / 16 exceeds the number of CUs, two feature tiles per
// workgroup (N % 32 == 0) finish in one round of workgroups instead of two.
//
// ROPE (FT == 2, N = (Hq + 2 Hkv) * 64: the QKV projection of a decode step): the two feature
// tiles of a workgroup are dims d..d+15 and d+32..d+47 of one head row, i.e. the partners of
// the half-split rotary embedding, and the epilogue does what rope_kv_write_kernel would do
// with the projection's bf16 output: rotate q and k rows by the token's position, store q
// rows to q_out and k / v rows into their cache slot (bf16 copy or fp8 quantisation), with
// the same arithmetic on the same bf16-rounded values, so the results are bit-identical to
// the two launches and the [T, N] intermediate never exists.

template <int TT, int FT, bool ROPE = false>
__global__ __launch_bounds__(kSkWaves * 64) void oproj_skinny_kernel(
    const uint16_t *__restrict__ a, const uint16_t *__restrict__ w,
    const uint16_t *__restrict__ bias, const uint16_t *resid,
    uint16_t *out, const int T, const int N, const int K, const RopeArgs rope = RopeArgs{}) {
  static_assert(!ROPE || FT == 2, "the rotation pairs two feature tiles");
  constexpr int kFtStride = ROPE ? 32 : 16;  // features between the workgroup's two tiles
  constexpr int kRows = TT * 16;
  constexpr int kLd = kRows / kSkWaves;  // slab rows per wave = loads per thread and slab
  constexpr int kTileBytes = kRows * kSkRowBytes;
  static_assert(2 * kTileBytes >= (int)sizeof(f32x4) * kSkWaves * TT * FT * 64, "reduction reuses the tiles");
  static_assert(TT * FT <= kSkWaves, "one wave per result tile in the epilogue");
  __shared__ __align__(16) uint8_t lds[2 * kTileBytes];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int n0 = ROPE ? (blockIdx.x >> 1) * 64 + (blockIdx.x & 1) * 16 : blockIdx.x * 16 * FT;
  const int nchunks = K / kSkChunk;
  const int R = (nchunks + kSkWaves - 1) / kSkWaves;

  const uint16_t *wp = w + (size_t)(n0 + i16) * K + g * 8;
  // slab loader: wave w fetches rows w, w + 8, ...; a lane 16 bytes of the row's 1 KiB
  const uint16_t *arow[kLd];
#pragma unroll
  for (int j = 0; j < kLd; ++j) arow[j] = a + (size_t)min(wave + kSkWaves * j, T - 1) * K;
  u32x4 ar[2][kLd];
  auto a_fetch = [&](const int st, const int r) {
    int col = r * kSkSlab + lane * 8;
    col = col < K ? col : 0;  // past the end of a short last slab: any valid address
#pragma unroll
    for (int j = 0; j < kLd; ++j) ar[st][j] = ld16(arow[j] + col);
  };
  const uint32_t st_off = (uint32_t)wave * kSkRowBytes + lane * 16;
  auto a_stash = [&](const int st, const int buf) {
#pragma unroll
    for (int j = 0; j < kLd; ++j)
      *(u32x4 *)(&lds[buf * kTileBytes + st_off + j * kSkWaves * kSkRowBytes]) = ar[st][j];
  };
  const uint32_t rd_off = (uint32_t)i16 * kSkRowBytes + wave * 128 + g * 16;

  f32x4 acc[FT][TT];
#pragma unroll
  for (int ft = 0; ft < FT; ++ft)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) acc[ft][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ROPE: what the epilogue needs from memory (position -> cos / sin row, cache slot) is
  // requested now by the waves that will need it, and has long arrived when the sums are done.
  f32x4 rope_c = {1.f, 1.f, 1.f, 1.f}, rope_s = {0.f, 0.f, 0.f, 0.f};
  int64_t rope_slot = -1;
  if constexpr (ROPE) {
    if (wave < TT) {
      const int t = min(wave * 16 + i16, T - 1);
      const int pos = min(max(rope.positions[t], 0), rope.max_pos - 1);
      const float *cs = rope.cos_sin + (size_t)pos * 64 + (n0 & 63) + 4 * g;
      rope_c = *(const f32x4 *)cs;
      rope_s = *(const f32x4 *)(cs + 32);
      rope_slot = rope.slot_mapping[t];
    }
  }

  // Rounds rb .. rb + 7.  Every load is issued unconditionally (clamped): a load under a
  // branch would leave the count of loads in flight unknown where the paths join, and the
  // waits that follow would then drain all of them.
  constexpr bool kEarlyW = TT < 4 && FT == 1;
  constexpr int kR = kSkRounds / FT;  // rounds per batch: 64 VGPRs of weights on their way
  Frag8 wf[kR][FT][2];
  auto w_fetch = [&](const int rb) {
#pragma unroll
    for (int j = 0; j < kR; ++j) {
      const int c = min((rb + j) * kSkWaves + wave, nchunks - 1);
#pragma unroll
      for (int ft = 0; ft < FT; ++ft) {
        wf[j][ft][0].u = ld16(wp + (size_t)ft * kFtStride * K + c * kSkChunk);
        wf[j][ft][1].u = ld16(wp + (size_t)ft * kFtStride * K + c * kSkChunk + 32);
      }
    }
  };
  auto batch = [&](const int rb) {
    if (rb > 0 || !kEarlyW) w_fetch(rb);  // else the first batch's weights are on their way
#pragma unroll
    for (int j = 0; j < kR; ++j) {
      const int par = j & 1;  // = (rb + j) % 2: rb is a multiple of kR, which is even
      const int r = rb + j;
      if (r >= R) break;  // (the same for every wave of the workgroup)
      // LDS tile `par` holds slab r, register stage par ^ 1 slab r + 1 (in flight)
      a_fetch(par, min(r + 2, R - 1));
      if (r * kSkWaves + wave < nchunks) {  // wave-uniform
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          Frag8 a0, a1;
          const uint8_t *src = &lds[par * kTileBytes + rd_off + tt * 16 * kSkRowBytes];
          a0.u = *(const u32x4 *)src;
          a1.u = *(const u32x4 *)(src + 64);
#pragma unroll
          for (int ft = 0; ft < FT; ++ft) {
            acc[ft][tt] = mfma16x32(wf[j][ft][0], a0, acc[ft][tt]);
            acc[ft][tt] = mfma16x32(wf[j][ft][1], a1, acc[ft][tt]);
          }
        }
      }
      a_stash(par ^ 1, par ^ 1);
      __syncthreads();
    }
  };

  // The weight stream should start before anything waits; with four token tiles the
  // registers do not stretch to holding it across the first slab's hand-over.
  a_fetch(0, 0);  // the small, cache-resident slab first: it gates the first round
  if (kEarlyW) w_fetch(0);
  a_fetch(1, min(1, R - 1));
  a_stash(0, 0);
  __syncthreads();
  if (R <= kR) {
    batch(0);  // straight-line code for K <= 4096
  } else {
    for (int rb = 0; rb < R; rb += kR) batch(rb);
  }

  f32x4(*red)[FT * TT][64] = reinterpret_cast<f32x4(*)[FT * TT][64]>(lds);  // all tile reads are done
#pragma unroll
  for (int ft = 0; ft < FT; ++ft)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) red[wave][ft * TT + tt][lane] = acc[ft][tt];
  __syncthreads();
  if constexpr (ROPE) {
    if (wave < TT) {  // wave tt: both tiles of token tile tt, rotation, stores
      f32x4 s1 = red[0][wave][lane], s2 = red[0][TT + wave][lane];
#pragma unroll
      for (int w2 = 1; w2 < kSkWaves; ++w2) {
        const f32x4 x = red[w2][wave][lane], y = red[w2][TT + wave][lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s1[e] += x[e];
          s2[e] += y[e];
        }
      }
      const int t = wave * 16 + i16;
      if (t >= T) return;
      const int head = n0 >> 6, d1 = (n0 & 63) + 4 * g;  // head row of [q | k | v], dim of s1[0]
      // the projection's output as eid_o_proj would have stored it: + bias, one bf16 rounding
      float x1[4], x2[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v1 = s1[e], v2 = s2[e];
        if (bias) {
          v1 += bf16_bits_to_f32(bias[n0 + 4 * g + e]);
          v2 += bf16_bits_to_f32(bias[n0 + 32 + 4 * g + e]);
        }
        x1[e] = bf16_bits_to_f32(pack_bf16(v1, 0.f) & 0xffffu);
        x2[e] = bf16_bits_to_f32(pack_bf16(v2, 0.f) & 0xffffu);
      }
      const bool is_v = head >= rope.Hq + rope.Hkv;
      float o1[4], o2[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        o1[e] = x1[e];
        o2[e] = x2[e];
      }
      if (!is_v) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o1[e] = __builtin_fmaf(-x2[e], rope_s[e], __fmul_rn(x1[e], rope_c[e]));
          o2[e] = __builtin_fmaf(x1[e], rope_s[e], __fmul_rn(x2[e], rope_c[e]));
        }
      }
      const u32x2 p1 = {pack_bf16(o1[0], o1[1]), pack_bf16(o1[2], o1[3])};
      const u32x2 p2 = {pack_bf16(o2[0], o2[1]), pack_bf16(o2[2], o2[3])};
      if (head < rope.Hq) {
        uint16_t *dst = rope.q_out + ((size_t)t * rope.Hq + head) * 64 + d1;
        *(u32x2 *)dst = p1;
        *(u32x2 *)(dst + 32) = p2;
        return;
      }
      const int64_t slot = rope_slot;
      if (slot < 0 || slot >= rope.num_slots) return;
      const int kh = is_v ? head - rope.Hq - rope.Hkv : head - rope.Hq;
      uint8_t *cache = is_v ? rope.v_cache : rope.k_cache;
      const size_t elem = ((size_t)slot * rope.Hkv + kh) * 64 + d1;
      if (rope.fp8) {
        const float sc = (is_v ? rope.v_scale : rope.k_scale)[kh];
        uint32_t q1 = 0, q2 = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float r1 = bf16_bits_to_f32((p1[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
          const float r2 = bf16_bits_to_f32((p2[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
          q1 |= fp8_e4m3_encode(__fdiv_rn(r1, sc)) << (e * 8);
          q2 |= fp8_e4m3_encode(__fdiv_rn(r2, sc)) << (e * 8);
        }
        *(uint32_t *)(cache + elem) = q1;
        *(uint32_t *)(cache + elem + 32) = q2;
      } else {
        *(u32x2 *)(cache + elem * 2) = p1;
        *(u32x2 *)(cache + (elem + 32) * 2) = p2;
      }
    }
    return;
  }
  if (wave < FT * TT) {  // wave (ft, tt) sums its tile over the eight K shares and writes it out
    f32x4 s = red[0][wave][lane];
#pragma unroll
    for (int w2 = 1; w2 < kSkWaves; ++w2) {
      const f32x4 x = red[w2][wave][lane];
      s[0] += x[0];
      s[1] += x[1];
      s[2] += x[2];
      s[3] += x[3];
    }
    const int ft = wave / TT, tt = wave - ft * TT;
    const int t = tt * 16 + i16;
    if (t < T) oproj_store(s, bias, resid, out, (size_t)t * N, n0 + ft * 16 + 4 * g);
  }
}

// ---------------------------------------------------------------------------------------
// Tiled kernel.  Workgroup = 4 waves = 128 tokens x 128 features; wave (wm, wn) owns a
// 64 x 64 quadrant (4 x 4 MFMA tiles).  K advances 64 elements per step; the next step's
// tiles travel global -> registers while the current ones are consumed from LDS, then
// registers -> LDS (rows padded to 144 bytes so that 16 lanes reading 16 bytes of 16 rows hit
// 16 distinct bank groups).
//
// Workgroup ids are dealt round-robin to the 8 XCDs by the hardware.  Ids are therefore
// remapped so that each XCD works through its own contiguous run of tiles, 8 token tiles
// deep: the 64 workgroups an XCD runs at a time share 8 activation and 8 weight tile rows
// through that XCD's L2.
// Requires K % 64 == 0 and N % 16 == 0.
// ---------------------------------------------------------------------------------------

// WF, WT = 16-row MFMA tiles per wave along features and tokens: 4, 4 gives the 128 x 128
// workgroup tile, 2, 2 a 64 x 64 one for batches too small to fill the device with the big tile
// (its K loop is as long, but four workgroups share a CU), 4, 2 128 features x 64 tokens.
// KT = K elements per step: 64, or 128 for the small tile (a loading instruction then covers
// 4 rows x 256 contiguous bytes instead of 8 rows x 128, and there are half as many steps,
// each of which is a round trip of loads, LDS stores and a barrier whatever it carries).
// SPLIT = 2: the workgroup is two such groups of 4 waves, each walking one half of K with LDS
// stages of its own (the barriers are the workgroup's, so the halves advance in step); at the
// end the second group hands its sums over through LDS and the first runs the epilogue.  For
// batches whose tiles do not fill the device (one workgroup per CU at most) this puts twice
// the loads in flight per CU and halves the number of steps, with no workspace and no
// reduction across workgroups.
template <int WF, int WT, int KT = 64, int SPLIT = 1>
__global__ __launch_bounds__(256 * SPLIT, SPLIT > 1 ? 1 : (WF == 4 || KT == 128) ? 2 : 4) void oproj_tiled_kernel(
    const uint16_t *__restrict__ a, const uint16_t *__restrict__ w,
    const uint16_t *__restrict__ bias, const uint16_t *resid,
    uint16_t *out, const int T, const int N, const int K, const int tiles_m,
    const int tiles_n) {
  // WF / WT = 16-row MFMA tiles per wave along the features / the tokens (2 x 2 waves)
  constexpr int kTileN = 32 * WF, kTileM = 32 * WT;  // rows of the workgroup tile
  constexpr int kWaveN = 16 * WF, kWaveM = 16 * WT;  // rows of a wave tile
  constexpr int kTlK = KT;
  constexpr int kTlRowBytes = 2 * KT + 16;  // (144 or 272 bytes: 16 lanes x 16 bytes of 16 rows on distinct banks)
  constexpr int kBytesN = kTileN * kTlRowBytes, kBytesM = kTileM * kTlRowBytes;
  constexpr int kSegs = KT / 8;             // 16-byte segments of a row
  constexpr int kRowsPerPass = 256 / kSegs; // rows the 256 threads cover with one load each
  constexpr int kPassesN = kTileN / kRowsPerPass, kPassesM = kTileM / kRowsPerPass;
  __shared__ __align__(16) uint8_t lds_w_all[SPLIT][2][kBytesN];
  __shared__ __align__(16) uint8_t lds_a_all[SPLIT][2][kBytesM];
  const int grp = SPLIT > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;  // which part of K
  uint8_t (*lds_w)[kBytesN] = lds_w_all[grp];
  uint8_t (*lds_a)[kBytesM] = lds_a_all[grp];
  const int tid = threadIdx.x & 255, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;

  // XCD-aware tile order: XCD x receives ids x, x + 8, ...; give it the contiguous run of
  // logical tiles [start_x, start_x + count_x), then walk the run in groups of 8 token tiles
  // (down the group first, then on to the next feature tile)
  const int total = tiles_m * tiles_n;
  const int xcd = blockIdx.x & 7, nth = blockIdx.x >> 3;
  const int logical = xcd * (total >> 3) + min(xcd, total & 7) + nth;
  const int group_size = 8 * tiles_n;
  const int first_m = (logical / group_size) * 8;
  const int rows = min(tiles_m - first_m, 8);
  const int in_group = logical % group_size;
  const int tm = first_m + in_group % rows, tn = in_group / rows;
  const int m0 = tm * kTileM, n0 = tn * kTileN;

  // loader: a wave instruction covers 8 rows x 128 bytes, or 4 rows x 256 (full lines)
  const int ld_row = tid / kSegs, ld_seg = tid % kSegs;  // rows ld_row + kRowsPerPass j
  const uint16_t *wsrc[kPassesN], *asrc[kPassesM];
#pragma unroll
  for (int j = 0; j < kPassesN; ++j)
    wsrc[j] = w + (size_t)min(n0 + ld_row + kRowsPerPass * j, N - 1) * K + ld_seg * 8 + grp * (K / SPLIT);
#pragma unroll
  for (int j = 0; j < kPassesM; ++j)
    asrc[j] = a + (size_t)min(m0 + ld_row + kRowsPerPass * j, T - 1) * K + ld_seg * 8 + grp * (K / SPLIT);
  const uint32_t st_off = (uint32_t)ld_row * kTlRowBytes + ld_seg * 16;
  f32x4 acc[WF][WT];  // [feature tile][token tile]
#pragma unroll
  for (int ft = 0; ft < WF; ++ft)
#pragma unroll
    for (int tt = 0; tt < WT; ++tt) acc[ft][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint32_t rd_w = (uint32_t)(wn * kWaveN + i16) * kTlRowBytes + g * 16;
  const uint32_t rd_a = (uint32_t)(wm * kWaveM + i16) * kTlRowBytes + g * 16;

  // Two register stages: the loads of K step i + 2 are issued while step i is computed and
  // are only needed (moved to LDS) at the end of step i + 1, so every global load has two
  // full steps to arrive.
  u32x4 wr[2][kPassesN], ar[2][kPassesM];
  auto fetch = [&](const int st, const int k0) {
#pragma unroll
    for (int j = 0; j < kPassesN; ++j) wr[st][j] = ld16(wsrc[j] + k0);
#pragma unroll
    for (int j = 0; j < kPassesM; ++j) ar[st][j] = ld16(asrc[j] + k0);
  };
  auto stash = [&](const int st, const int buf) {
#pragma unroll
    for (int j = 0; j < kPassesN; ++j) *(u32x4 *)(&lds_w[buf][st_off + j * kRowsPerPass * kTlRowBytes]) = wr[st][j];
#pragma unroll
    for (int j = 0; j < kPassesM; ++j) *(u32x4 *)(&lds_a[buf][st_off + j * kRowsPerPass * kTlRowBytes]) = ar[st][j];
  };
  const int nk = K / SPLIT / kTlK;
  auto step = [&](const int par, const int i) {  // par = i % 2, a literal at both call sites
    // unconditional (the last steps refetch the final slab and never use it): a fetch under
    // a branch would leave the number of loads in flight unknown at the join and force the
    // LDS stores below to wait for all of them
    fetch(par, min(i + 2, nk - 1) * kTlK);
#pragma unroll
    for (int ks = 0; ks < KT / 32; ++ks) {
      Frag8 wf[WF], af[WT];
#pragma unroll
      for (int x = 0; x < WF; ++x) wf[x].u = *(const u32x4 *)(&lds_w[par][rd_w + x * 16 * kTlRowBytes + ks * 64]);
#pragma unroll
      for (int x = 0; x < WT; ++x) af[x].u = *(const u32x4 *)(&lds_a[par][rd_a + x * 16 * kTlRowBytes + ks * 64]);
#pragma unroll
      for (int ft = 0; ft < WF; ++ft)
#pragma unroll
        for (int tt = 0; tt < WT; ++tt) acc[ft][tt] = mfma16x32(wf[ft], af[tt], acc[ft][tt]);
    }
    if (i + 1 < nk) stash(par ^ 1, par ^ 1);
    __syncthreads();
  };

  fetch(0, 0);
  fetch(1, min(1, nk - 1) * kTlK);
  stash(0, 0);
  __syncthreads();
  for (int i = 0; i < nk; i += 2) {
    step(0, i);
    if (i + 1 < nk) step(1, i + 1);
  }

  if constexpr (SPLIT > 1) {
    // (every wave is past the last step's barrier: the stages are free) the other groups' sums ->
    // LDS (each into its own stages: the weight stages first, then the activation stages) ->
    // first group, added in group order
    constexpr int kInW = 2 * kBytesN / 4096, kInA = 2 * kBytesM / 4096;  // tiles of 256 x 16 bytes
    static_assert(WF * WT <= kInW + kInA, "a group's sums fit its stages");
    auto cell = [&](const int gg, const int idx) {
      return idx < kInW ? reinterpret_cast<f32x4 *>(&lds_w_all[gg][0][0]) + idx * 256 + tid
                        : reinterpret_cast<f32x4 *>(&lds_a_all[gg][0][0]) + (idx - kInW) * 256 + tid;
    };
    if (grp > 0) {
#pragma unroll
      for (int ft = 0; ft < WF; ++ft)
#pragma unroll
        for (int tt = 0; tt < WT; ++tt) *cell(grp, ft * WT + tt) = acc[ft][tt];
    }
    __syncthreads();
    if (grp > 0) return;
#pragma unroll
    for (int gg = 1; gg < SPLIT; ++gg) {
#pragma unroll
      for (int ft = 0; ft < WF; ++ft)
#pragma unroll
        for (int tt = 0; tt < WT; ++tt) {
          const f32x4 o = *cell(gg, ft * WT + tt);
          acc[ft][tt] = f32x4{acc[ft][tt][0] + o[0], acc[ft][tt][1] + o[1], acc[ft][tt][2] + o[2], acc[ft][tt][3] + o[3]};
        }
    }
  }
  oproj_epilogue<WF, WT>(acc, bias, resid, out, T, N, m0 + wm * kWaveM + i16, n0 + wn * kWaveN + 4 * g);
}

// ---------------------------------------------------------------------------------------
// Wide kernel (prefill-sized batches).  OCC workgroups per CU; workgroup tile = 16 WT WM tokens
// x 16 WF WN features, wave (wm, wn) owns 16 WT tokens x 16 WF features.  K advances 64
// elements per step through two LDS stages that the loads fill directly
// (global_load_lds_dwordx4: a wave instruction moves 8 rows x 128 bytes, no registers), the
// eight 16-byte segments of a row permuted by (row / 2) % 8 so that fragment reads are free of
// bank conflicts.  One barrier per step, placed between its two 32-element halves: by then the
// stage of the next step has had a whole step to arrive, the first half's fragments of the
// next step are fetched from LDS while the second half's MFMAs run, and the stage just
// finished is handed to the loads of the step after next.
// Requires K % 64 == 0 and N % 16 == 0.
// ---------------------------------------------------------------------------------------
namespace {
typedef __attribute__((address_space(1))) const void dma_gptr_t;
typedef __attribute__((address_space(3))) void dma_lptr_t;
}  // namespace

template <int WF, int WT, int WN, int WM, int OCC>
__global__ __launch_bounds__(64 * WN * WM, OCC) void oproj_wide_kernel(
    const uint16_t *__restrict__ a, const uint16_t *__restrict__ w,
    const uint16_t *__restrict__ bias, const uint16_t *resid,
    uint16_t *out, const int T, const int N, const int K, const int tiles_m,
    const int tiles_n) {
  constexpr int kNF = 16 * WF * WN, kNT = 16 * WT * WM, kWaves = WN * WM;
  constexpr int kRows = kNF + kNT, kStage = kRows * 128;
  constexpr int kPieces = kRows / 8;  // 1 KiB pieces of a stage
  static_assert(kPieces % kWaves == 0 && kNF % 16 == 0, "pieces are dealt evenly to the waves");
  constexpr int kPer = kPieces / kWaves;
  __shared__ __align__(1024) uint8_t stage0[kStage];
  __shared__ __align__(1024) uint8_t stage1[kStage];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;

  // XCD-aware tile order, as in the tiled kernel
  const int total = tiles_m * tiles_n;
  const int xcd = blockIdx.x & 7, nth = blockIdx.x >> 3;
  const int logical = xcd * (total >> 3) + min(xcd, total & 7) + nth;
  const int group_size = 8 * tiles_n;
  const int first_m = (logical / group_size) * 8;
  const int rows = min(tiles_m - first_m, 8);
  const int in_group = logical % group_size;
  const int tm = first_m + in_group % rows, tn = in_group / rows;
  const int m0 = tm * kNT, n0 = tn * kNF;

  // loader: piece p = wave + kWaves j covers stage rows 8 p .. 8 p + 7 (weight rows first, then
  // token rows); lane (r, s) = (lane / 8, lane % 8) fills slot s of row r with the row's
  // segment s ^ ((row / 2) % 8)
  const uint16_t *src[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int row = (wave + kWaves * j) * 8 + (lane >> 3);
    const int seg = (lane & 7) ^ ((row >> 1) & 7);  // (kNF % 16 == 0: the same for either part)
    src[j] = row < kNF ? w + (size_t)min(n0 + row, N - 1) * K + seg * 8
                       : a + (size_t)min(m0 + row - kNF, T - 1) * K + seg * 8;
  }
  auto dma = [&](uint8_t *stage, const int k0) {
#pragma unroll
    for (int j = 0; j < kPer; ++j)
      __builtin_amdgcn_global_load_lds((dma_gptr_t *)(src[j] + k0),
                                       (dma_lptr_t *)(stage + (wave + kWaves * j) * 1024), 16, 0, 0);
  };
  // reader: lane (i16, g) wants segment 4 half + g of row i16 of a 16-row tile
  const uint32_t slot = (uint32_t)(g ^ ((i16 >> 1) & 7));
  const uint32_t rd_w = (uint32_t)(wn * 16 * WF + i16) * 128 + slot * 16;
  const uint32_t rd_a = (uint32_t)(kNF + wm * 16 * WT + i16) * 128 + slot * 16;
  auto read = [&](const uint8_t *stage, const int half, Frag8 (&wf)[WF], Frag8 (&af)[WT]) {
#pragma unroll
    for (int x = 0; x < WF; ++x) wf[x].u = *(const u32x4 *)(stage + ((rd_w + x * 2048) ^ (half * 64)));
#pragma unroll
    for (int x = 0; x < WT; ++x) af[x].u = *(const u32x4 *)(stage + ((rd_a + x * 2048) ^ (half * 64)));
  };
  f32x4 acc[WF][WT];
#pragma unroll
  for (int ft = 0; ft < WF; ++ft)
#pragma unroll
    for (int tt = 0; tt < WT; ++tt) acc[ft][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto mfmas = [&](const Frag8 (&wf)[WF], const Frag8 (&af)[WT]) {
#pragma unroll
    for (int ft = 0; ft < WF; ++ft)
#pragma unroll
      for (int tt = 0; tt < WT; ++tt) acc[ft][tt] = mfma16x32(wf[ft], af[tt], acc[ft][tt]);
  };

  const int nk = K / 64;
  Frag8 wf0[WF], af0[WT], wf1[WF], af1[WT];
  auto step = [&](uint8_t *cur, uint8_t *nxt, const int i) {
    read(cur, 1, wf1, af1);
    mfmas(wf0, af0);
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0), lgkmcnt(0): my share of step i + 1 has landed, my reads of `cur` are done
    __syncthreads();
    if (i + 2 < nk) dma(cur, (i + 2) * 64);
    read(nxt, 0, wf0, af0);  // (in the last step: a stage nobody needs, still this workgroup's memory)
    mfmas(wf1, af1);
  };
  dma(stage0, 0);
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();
  if (nk > 1) dma(stage1, 64);
  read(stage0, 0, wf0, af0);
  for (int i = 0; i < nk; i += 2) {
    step(stage0, stage1, i);
    if (i + 1 < nk) step(stage1, stage0, i + 1);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // no load may still be writing this workgroup's LDS when it ends

  oproj_epilogue<WF, WT>(acc, bias, resid, out, T, N, m0 + wm * 16 * WT + i16, n0 + wn * 16 * WF + 4 * g);
}

int device_cus();  // attn_kernels.hip

hipError_t launch_o_proj(const uint16_t *a, const uint16_t *w, const uint16_t *bias,
                         const uint16_t *resid, uint16_t *out, int T, int N, int K,
                         hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (T <= 64) {
    const dim3 block(kSkWaves * 64);
    // one workgroup per CU (registers, LDS): no more workgroups than CUs if that can be had
    if (N / 16 > device_cus() && N % 32 == 0) {
      const dim3 grid(N / 32);
      if (T <= 16)
        oproj_skinny_kernel<1, 2><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
      else if (T <= 32)
        oproj_skinny_kernel<2, 2><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
      else if (T <= 48)
        oproj_skinny_kernel<3, 2><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
      else
        oproj_skinny_kernel<4, 2><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
      return hipGetLastError();
    }
    const dim3 grid(N / 16);
    if (T <= 16)
      oproj_skinny_kernel<1, 1><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    else if (T <= 32)
      oproj_skinny_kernel<2, 1><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    else if (T <= 48)
      oproj_skinny_kernel<3, 1><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    else
      oproj_skinny_kernel<4, 1><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    return hipGetLastError();
  }
  // Which tiling?  Every kernel covers the output in rounds of workgroups, and a workgroup that
  // walks all of K takes about as long whatever its tile (the K steps' load latency): measured
  // for 2880 x 4096, a round of the 256 x 192 kernel (one workgroup per CU) takes ~85 us and a
  // round of the direct-to-LDS 128 x 128 kernel (two per CU) ~63 us.  The cheaper plan wins.
  // Batches whose tiles give at most one workgroup per CU take the register-staged kernel with
  // the two halves of K side by side in one workgroup.  Such a workgroup is bound by what its CU
  // takes in per unit of time (~48 GB/s of tile rows, whatever the tile), i.e. by
  // K x (tile features + tile tokens) bytes: of the tiles that cover the output with no more
  // workgroups than CUs (features x tokens: 64 x 64, 96 x 64, 128 x 64, 96 x 128, 128 x 128) the
  // one with the smallest sum is taken.
  // EID_OPROJ_KERNEL=wide|mid|tiled overrides the choice (tests, measurements); "tiled" is the
  // register-staged kernel; EID_OPROJ_NOSPLIT=1 and EID_OPROJ_K64=1 take its earlier forms (one
  // group of four waves; K in steps of 64) for A/B measurements.
  const int cus = device_cus();
  static const bool k64 = getenv("EID_OPROJ_K64") != nullptr;
  static const bool nosplit = getenv("EID_OPROJ_NOSPLIT") != nullptr;
  const long t64 = (long)((T + 63) / 64) * ((N + 63) / 64);
  const long tb = (long)((T + 127) / 128) * ((N + 127) / 128);
  struct Cand { int nf, nt; };
  static const Cand cands[5] = {{64, 64}, {96, 64}, {128, 64}, {96, 128}, {128, 128}};
  int best = -1;
  for (int c = 0; c < 5; ++c) {
    const long cnt = (long)((T + cands[c].nt - 1) / cands[c].nt) * ((N + cands[c].nf - 1) / cands[c].nf);
    if (cnt <= cus && (best < 0 || cands[c].nf + cands[c].nt < cands[best].nf + cands[best].nt)) best = c;
  }
  const long tw = (long)((T + 255) / 256) * ((N + 191) / 192);
  const double wide_cost = (double)((tw + cus - 1) / cus) * 85.0;
  const double mid_cost = (double)((tb + 2 * cus - 1) / (2 * cus)) * 63.0;
  int plan = 4 * tb < 3 * cus ? 0 : wide_cost < mid_cost ? 2 : 1;  // 0 = register-staged tiles, 1 = mid, 2 = wide
  const bool split_ok = K % 256 == 0 && !k64 && !nosplit && best >= 0;
  if (split_ok) plan = 0;
  if (const char *e = getenv("EID_OPROJ_KERNEL")) plan = e[0] == 'w' ? 2 : e[0] == 'm' ? 1 : e[0] == 't' ? 0 : plan;
  if (plan == 2) {
    const int tiles_m = (T + 255) / 256, tiles_n = (N + 191) / 192;
    oproj_wide_kernel<6, 4, 2, 4, 1><<<tiles_m * tiles_n, 512, 0, st>>>(a, w, bias, resid, out, T, N, K,
                                                                       tiles_m, tiles_n);
    return hipGetLastError();
  }
  if (plan == 1) {
    const int tiles_m = (T + 127) / 128, tiles_n = (N + 127) / 128;
    oproj_wide_kernel<4, 4, 2, 2, 2><<<tiles_m * tiles_n, 256, 0, st>>>(a, w, bias, resid, out, T, N, K,
                                                                       tiles_m, tiles_n);
    return hipGetLastError();
  }
  if (plan == 0 && split_ok) {
    const int tm = (T + cands[best].nt - 1) / cands[best].nt, tn = (N + cands[best].nf - 1) / cands[best].nf;
    const unsigned grid = (unsigned)(tm * tn);
    switch (best) {  // (256 tokens: 35.1 us with steps of 64, 26.3 with steps of 128, 22.5 split)
      case 0: oproj_tiled_kernel<2, 2, 128, 2><<<grid, 512, 0, st>>>(a, w, bias, resid, out, T, N, K, tm, tn); break;
      case 1: oproj_tiled_kernel<3, 2, 64, 2><<<grid, 512, 0, st>>>(a, w, bias, resid, out, T, N, K, tm, tn); break;
      case 2: oproj_tiled_kernel<4, 2, 64, 2><<<grid, 512, 0, st>>>(a, w, bias, resid, out, T, N, K, tm, tn); break;
      case 3: oproj_tiled_kernel<3, 4, 64, 2><<<grid, 512, 0, st>>>(a, w, bias, resid, out, T, N, K, tm, tn); break;
      default: oproj_tiled_kernel<4, 4, 64, 2><<<grid, 512, 0, st>>>(a, w, bias, resid, out, T, N, K, tm, tn); break;
    }
  } else if (4 * tb >= 3 * cus) {
    // the 128 x 128 tile once it gives most CUs a workgroup, else 64 x 64
    oproj_tiled_kernel<4, 4><<<(unsigned)tb, 256, 0, st>>>(a, w, bias, resid, out, T, N, K, (T + 127) / 128,
                                                          (N + 127) / 128);
  } else if (K % 128 == 0 && !k64) {
    oproj_tiled_kernel<2, 2, 128><<<(unsigned)t64, 256, 0, st>>>(a, w, bias, resid, out, T, N, K, (T + 63) / 64,
                                                                (N + 63) / 64);
  } else {
    oproj_tiled_kernel<2, 2><<<(unsigned)t64, 256, 0, st>>>(a, w, bias, resid, out, T, N, K, (T + 63) / 64,
                                                           (N + 63) / 64);
  }
  return hipGetLastError();
}

// QKV projection + rotary embedding + split + KV write in one launch (decode batches).
hipError_t launch_qkv_rope(const uint16_t *a, const uint16_t *w, const uint16_t *bias, int T, int K,
                           const RopeArgs &r, hipStream_t st) {
  if (T == 0) return hipSuccess;
  const int N = (r.Hq + 2 * r.Hkv) * 64;
  const dim3 grid(N / 32), block(kSkWaves * 64);
  if (T <= 16)
    oproj_skinny_kernel<1, 2, true><<<grid, block, 0, st>>>(a, w, bias, nullptr, nullptr, T, N, K, r);
  else if (T <= 32)
    oproj_skinny_kernel<2, 2, true><<<grid, block, 0, st>>>(a, w, bias, nullptr, nullptr, T, N, K, r);
  else if (T <= 48)
    oproj_skinny_kernel<3, 2, true><<<grid, block, 0, st>>>(a, w, bias, nullptr, nullptr, T, N, K, r);
  else
    oproj_skinny_kernel<4, 2, true><<<grid, block, 0, st>>>(a, w, bias, nullptr, nullptr, T, N, K, r);
  return hipGetLastError();
}

}  // namespace eid
