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
// Two kernels:
//   oproj_skinny_kernel  T <= 64 (decode batches).  HBM-bound: the weight (N*K*2 bytes) is
//                        streamed once.  One workgroup per 16 features; its 8 waves deal the
//                        K dimension in 64-element chunks, each wave keeps a whole batch of
//                        weight loads in flight, the partial sums meet in LDS.
//   oproj_tiled_kernel   any T.  MFMA-bound: 128 tokens x 128 features per workgroup, K in
//                        steps of 64 through double-buffered, row-padded LDS tiles.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "eid_device.h"

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

constexpr int kSkWaves = 8;
constexpr int kSkChunk = 64;   // K elements per chunk: one 128-byte line of every weight row
constexpr int kSkBatch = 8;    // chunks whose weight loads a wave issues back to back

}  // namespace

// ---------------------------------------------------------------------------------------
// Skinny kernel.  grid = N / 16, block = 512.  TT = number of 16-token tiles (T <= 16 TT).
// Wave w takes chunks w, w + 8, w + 16, ... of the K dimension.  Requires K % 64 == 0.
// ---------------------------------------------------------------------------------------
template <int TT>
__global__ __launch_bounds__(kSkWaves * 64) void oproj_skinny_kernel(
    const uint16_t *__restrict__ a, const uint16_t *__restrict__ w,
    const uint16_t *__restrict__ bias, const uint16_t *resid,
    uint16_t *out, const int T, const int N, const int K) {
  __shared__ f32x4 red[kSkWaves][TT][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nchunks = K / kSkChunk;

  const uint16_t *wp = w + (size_t)(n0 + i16) * K + g * 8;
  const uint16_t *ap[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) ap[tt] = a + (size_t)min(tt * 16 + i16, T - 1) * K + g * 8;

  f32x4 acc[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) acc[tt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int c0 = wave; c0 < nchunks; c0 += kSkWaves * kSkBatch) {
    // the whole batch of weight fragments first: 2 KiB per chunk and wave in flight
    Frag8 wf[kSkBatch][2];
#pragma unroll
    for (int j = 0; j < kSkBatch; ++j) {
      const int c = min(c0 + j * kSkWaves, nchunks - 1);  // a repeated chunk is skipped below
      wf[j][0].u = ld16(wp + c * kSkChunk);
      wf[j][1].u = ld16(wp + c * kSkChunk + 32);
    }
#pragma unroll
    for (int j = 0; j < kSkBatch; ++j) {
      const int c = c0 + j * kSkWaves;
      if (c < nchunks) {  // wave-uniform
        Frag8 af[TT][2];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          af[tt][0].u = ld16(ap[tt] + c * kSkChunk);
          af[tt][1].u = ld16(ap[tt] + c * kSkChunk + 32);
        }
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          acc[tt] = mfma16x32(wf[j][0], af[tt][0], acc[tt]);
          acc[tt] = mfma16x32(wf[j][1], af[tt][1], acc[tt]);
        }
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) red[wave][tt][lane] = acc[tt];
  __syncthreads();
  if (wave < TT) {  // wave tt sums tile tt over the eight K shares and writes it out
    f32x4 s = red[0][wave][lane];
#pragma unroll
    for (int w2 = 1; w2 < kSkWaves; ++w2) {
      const f32x4 x = red[w2][wave][lane];
      s[0] += x[0];
      s[1] += x[1];
      s[2] += x[2];
      s[3] += x[3];
    }
    const int t = wave * 16 + i16;
    if (t < T) oproj_store(s, bias, resid, out, (size_t)t * N, n0 + 4 * g);
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
namespace {
constexpr int kTlTile = 128;
constexpr int kTlK = 64;
constexpr int kTlRowBytes = 144;
constexpr int kTlTileBytes = kTlTile * kTlRowBytes;
}  // namespace

__global__ __launch_bounds__(256, 2) void oproj_tiled_kernel(
    const uint16_t *__restrict__ a, const uint16_t *__restrict__ w,
    const uint16_t *__restrict__ bias, const uint16_t *resid,
    uint16_t *out, const int T, const int N, const int K, const int tiles_m,
    const int tiles_n) {
  __shared__ __align__(16) uint8_t lds_w[2][kTlTileBytes];
  __shared__ __align__(16) uint8_t lds_a[2][kTlTileBytes];
  const int tid = threadIdx.x, lane = tid & 63;
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
  const int m0 = tm * kTlTile, n0 = tn * kTlTile;

  // loader: a wave instruction covers 8 rows x 128 bytes (full lines)
  const int ld_row = tid >> 3, ld_seg = tid & 7;  // rows ld_row + 32 j
  const uint16_t *wsrc[4], *asrc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    wsrc[j] = w + (size_t)min(n0 + ld_row + 32 * j, N - 1) * K + ld_seg * 8;
    asrc[j] = a + (size_t)min(m0 + ld_row + 32 * j, T - 1) * K + ld_seg * 8;
  }
  const uint32_t st_off = (uint32_t)ld_row * kTlRowBytes + ld_seg * 16;
  u32x4 wr[4], ar[4];
  auto fetch = [&](const int k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      wr[j] = ld16(wsrc[j] + k0);
      ar[j] = ld16(asrc[j] + k0);
    }
  };
  auto stash = [&](const int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      *(u32x4 *)(&lds_w[buf][st_off + j * 32 * kTlRowBytes]) = wr[j];
      *(u32x4 *)(&lds_a[buf][st_off + j * 32 * kTlRowBytes]) = ar[j];
    }
  };

  f32x4 acc[4][4];  // [feature tile][token tile]
#pragma unroll
  for (int ft = 0; ft < 4; ++ft)
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) acc[ft][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint32_t rd_w = (uint32_t)(wn * 64 + i16) * kTlRowBytes + g * 16;
  const uint32_t rd_a = (uint32_t)(wm * 64 + i16) * kTlRowBytes + g * 16;

  fetch(0);
  stash(0);
  __syncthreads();
  int cur = 0;
  for (int k0 = 0; k0 < K; k0 += kTlK, cur ^= 1) {
    const bool has_next = k0 + kTlK < K;
    if (has_next) fetch(k0 + kTlK);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      Frag8 wf[4], af[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        wf[i].u = *(const u32x4 *)(&lds_w[cur][rd_w + i * 16 * kTlRowBytes + ks * 64]);
        af[i].u = *(const u32x4 *)(&lds_a[cur][rd_a + i * 16 * kTlRowBytes + ks * 64]);
      }
#pragma unroll
      for (int ft = 0; ft < 4; ++ft)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) acc[ft][tt] = mfma16x32(wf[ft], af[tt], acc[ft][tt]);
    }
    if (has_next) stash(cur ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int tt = 0; tt < 4; ++tt) {
    const int t = m0 + wm * 64 + tt * 16 + i16;
    if (t >= T) continue;
#pragma unroll
    for (int ft = 0; ft < 4; ++ft) {
      const int n = n0 + wn * 64 + ft * 16 + 4 * g;
      if (n < N) oproj_store(acc[ft][tt], bias, resid, out, (size_t)t * N, n);
    }
  }
}

hipError_t launch_o_proj(const uint16_t *a, const uint16_t *w, const uint16_t *bias,
                         const uint16_t *resid, uint16_t *out, int T, int N, int K,
                         hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (T <= 64) {
    const dim3 grid(N / 16), block(kSkWaves * 64);
    if (T <= 16)
      oproj_skinny_kernel<1><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    else if (T <= 32)
      oproj_skinny_kernel<2><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    else if (T <= 48)
      oproj_skinny_kernel<3><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    else
      oproj_skinny_kernel<4><<<grid, block, 0, st>>>(a, w, bias, resid, out, T, N, K);
    return hipGetLastError();
  }
  const int tiles_m = (T + kTlTile - 1) / kTlTile, tiles_n = (N + kTlTile - 1) / kTlTile;
  oproj_tiled_kernel<<<tiles_m * tiles_n, 256, 0, st>>>(a, w, bias, resid, out, T, N, K, tiles_m,
                                                       tiles_n);
  return hipGetLastError();
}

}  // namespace eid
