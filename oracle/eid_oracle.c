/*
 * eid_oracle.c — CPU oracle for the paged sink-attention path (see eid_oracle.h).
 * TEST INFRASTRUCTURE ONLY.  No reference source exists for this path
 * (eidola-ai/eidola proxies inference: docs/server.md:102-109), so each function
 * follows the mathematical definition stated next to it; parity with the reference
 * is unpinned, parity with the definition is pinned by tests/test_oracle_*.py.
 */
#include "eid_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ conversions */

float orc_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* bf16 = upper 16 bits of fp32 after round-to-nearest-even on the dropped 16 bits. */
uint16_t orc_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* Nearest bf16 to a double, ties to even, decided in double arithmetic: the two bf16
 * neighbours of x are found from its fp32 truncation, so no second rounding intervenes. */
uint16_t orc_f64_to_bf16(double x) {
  if (isnan(x)) return 0x7FC0u;
  const double ax = fabs(x);
  const uint16_t sign = signbit(x) ? 0x8000u : 0u;
  if (ax >= 3.3961775292304225e38) return (uint16_t)(sign | 0x7F80u); /* >= max + half ulp */
  /* largest bf16 magnitude <= ax: search by bits (monotone for non-negative values) */
  uint32_t lo = 0, hi = 0x7F7Fu;
  while (lo < hi) {
    const uint32_t mid = (lo + hi + 1) >> 1;
    if ((double)orc_bf16_to_f32((uint16_t)mid) <= ax) lo = mid; else hi = mid - 1;
  }
  const double below = (double)orc_bf16_to_f32((uint16_t)lo);
  if (below == ax || lo == 0x7F7Fu) return (uint16_t)(sign | lo);
  const double above = (double)orc_bf16_to_f32((uint16_t)(lo + 1));
  const double d_lo = ax - below, d_hi = above - ax; /* exact: neighbours within a factor 2 */
  uint32_t pick = d_lo < d_hi ? lo : d_hi < d_lo ? lo + 1 : ((lo & 1u) ? lo + 1 : lo);
  return (uint16_t)(sign | pick);
}

/* OCP e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; S.1111.111 = NaN;
 * largest finite 448 = 1.75 * 2^8; subnormals are multiples of 2^-9. */
float orc_fp8_e4m3_decode(uint8_t b) {
  int s = b >> 7, e = (b >> 3) & 0xF, m = b & 7;
  float v;
  if (e == 0xF && m == 7) return NAN;
  if (e == 0)
    v = ldexpf((float)m, -9);
  else
    v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return s ? -v : v;
}

/* Round-to-nearest-even onto the e4m3fn grid, saturating at +-448.  Works on the grid
 * spacing directly: for |x| in [2^e, 2^(e+1)) with e >= -6 the spacing is 2^(e-3); below
 * 2^-6 the spacing is 2^-9.  nearbyint() in the default rounding mode is RNE. */
uint8_t orc_fp8_e4m3_encode(float x) {
  if (isnan(x)) return 0x7F;
  uint8_t sign = signbit(x) ? 0x80 : 0x00;
  double a = fabs((double)x);
  if (a >= 448.0) return (uint8_t)(sign | 0x7E);
  int e;
  (void)frexp(a, &e); /* a = f * 2^e, f in [0.5,1)  =>  a in [2^(e-1), 2^e) */
  int ex = e - 1;
  if (a == 0.0 || ex < -6) ex = -6;
  double q = ldexp(1.0, ex - 3);     /* grid spacing */
  double n = nearbyint(a / q);       /* integer multiple, RNE; exact division by 2^k */
  /* n in [0,16]; n == 16 means we rounded up into the next binade */
  if (ex == -6 && n < 8.0) return (uint8_t)(sign | (uint8_t)n); /* subnormal or zero */
  if (n >= 16.0) {
    ex += 1;
    n = 8.0;
  }
  int E = ex + 7, M = (int)n - 8;
  if (E > 15 || (E == 15 && M > 6)) return (uint8_t)(sign | 0x7E);
  return (uint8_t)(sign | (E << 3) | M);
}

/* ------------------------------------------------------------------ helpers */

static inline double kv_elem(const void *cache, int kv_dtype, size_t idx) {
  if (kv_dtype == EID_KV_FP8_E4M3) return (double)orc_fp8_e4m3_decode(((const uint8_t *)cache)[idx]);
  return (double)orc_bf16_to_f32(((const uint16_t *)cache)[idx]);
}

/* A query row at absolute position p sees keys max(0, p-W+1)..p (W = 0: 0..p). */
static inline int32_t first_key(int32_t p, int32_t W) {
  if (W <= 0) return 0;
  int32_t lo = p - W + 1;
  return lo < 0 ? 0 : lo;
}

int32_t orc_kv_begin(int32_t seq_len, int32_t q_len, int32_t window, int32_t block_size) {
  int32_t p0 = seq_len - q_len; /* position of the first query row */
  if (p0 < 0) p0 = 0;
  int32_t lo = first_key(p0, window);
  return lo - lo % block_size;
}

static inline void seq_rows(const eid_attn_desc *d, const eid_attn_args *a, int s, int *row0,
                            int *qlen) {
  if (a->cu_seqlens_q) {
    *row0 = a->cu_seqlens_q[s];
    *qlen = a->cu_seqlens_q[s + 1] - a->cu_seqlens_q[s];
  } else {
    *row0 = s;
    *qlen = 1;
  }
  (void)d;
}

/* ------------------------------------------------------------------ K1 */

/* cache_flat[slot, h, :] = f(new[t, h, :]); slot < 0 skipped.
 * fp8: f(x) = RNE_e4m3fn(clamp(fp32(x) / scale[h], -448, 448)) with IEEE fp32 division. */
int orc_kv_write(const eid_attn_desc *d, const uint16_t *k_new, const uint16_t *v_new,
                 void *k_cache, void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                 const float *k_scale, const float *v_scale) {
  const int H = d->num_kv_heads, D = d->head_dim;
  const int64_t nslots = d->num_blocks * d->block_size;
  for (int t = 0; t < num_tokens; t++) {
    int64_t slot = slot_mapping[t];
    if (slot < 0) continue;
    if (slot >= nslots) return -1;
    for (int h = 0; h < H; h++)
      for (int x = 0; x < D; x++) {
        size_t src = ((size_t)t * H + h) * D + x;
        size_t dst = ((size_t)slot * H + h) * D + x;
        if (d->kv_dtype == EID_KV_FP8_E4M3) {
          volatile float kq = orc_bf16_to_f32(k_new[src]) / k_scale[h];
          volatile float vq = orc_bf16_to_f32(v_new[src]) / v_scale[h];
          ((uint8_t *)k_cache)[dst] = orc_fp8_e4m3_encode(kq);
          ((uint8_t *)v_cache)[dst] = orc_fp8_e4m3_encode(vq);
        } else {
          ((uint16_t *)k_cache)[dst] = k_new[src];
          ((uint16_t *)v_cache)[dst] = v_new[src];
        }
      }
  }
  return 0;
}

/* Fused rotary embedding + QKV split + KV write: same contract as eid_rope_kv_write
 * (include/eidola_attn.h).  Half-split pairing (dim i with dim i + D/2); per pair, in fp32,
 *   o1 = fma(-x2, sin, x1 * cos),  o2 = fma(x1, sin, x2 * cos),  each rounded to bf16 RNE;
 * the rotated k row and the v row then go through orc_kv_write's rule.  Reference
 * counterpart: none (the reference holds no model code).  `volatile` keeps the product a
 * separately rounded fp32 value whatever the compiler's contraction settings are. */
int orc_rope_kv_write(const eid_attn_desc *d, const uint16_t *qkv, const int32_t *positions,
                      const float *cos_sin, int32_t max_pos, uint16_t *q_out, void *k_cache,
                      void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                      const float *k_scale, const float *v_scale) {
  const int Hq = d->num_q_heads, Hkv = d->num_kv_heads, D = d->head_dim, half = D / 2;
  const int64_t nslots = d->num_blocks * d->block_size;
  const size_t row = (size_t)(Hq + 2 * Hkv) * D;
  for (int t = 0; t < num_tokens; t++) {
    int pos = positions[t];
    if (pos < 0) pos = 0;
    if (pos > max_pos - 1) pos = max_pos - 1;
    const float *cs = cos_sin + (size_t)pos * D;
    const int64_t slot = slot_mapping[t];
    if (slot >= nslots) return -1;
    for (int h = 0; h < Hq + 2 * Hkv; h++) {
      const uint16_t *src = qkv + (size_t)t * row + (size_t)h * D;
      uint16_t o[256];
      if (h < Hq + Hkv) {
        for (int i = 0; i < half; i++) {
          const float x1 = orc_bf16_to_f32(src[i]), x2 = orc_bf16_to_f32(src[i + half]);
          volatile float p1 = x1 * cs[i], p2 = x2 * cs[i];
          o[i] = orc_f32_to_bf16(fmaf(-x2, cs[half + i], p1));
          o[i + half] = orc_f32_to_bf16(fmaf(x1, cs[half + i], p2));
        }
      } else {
        memcpy(o, src, (size_t)D * sizeof(uint16_t));
      }
      if (h < Hq) {
        memcpy(q_out + ((size_t)t * Hq + h) * D, o, (size_t)D * sizeof(uint16_t));
        continue;
      }
      if (slot < 0) continue;
      const int is_v = h >= Hq + Hkv;
      const int kh = is_v ? h - Hq - Hkv : h - Hq;
      void *cache = is_v ? v_cache : k_cache;
      const float *scale = is_v ? v_scale : k_scale;
      for (int x = 0; x < D; x++) {
        const size_t dst = ((size_t)slot * Hkv + kh) * D + x;
        if (d->kv_dtype == EID_KV_FP8_E4M3) {
          volatile float qv = orc_bf16_to_f32(o[x]) / scale[kh];
          ((uint8_t *)cache)[dst] = orc_fp8_e4m3_encode(qv);
        } else {
          ((uint16_t *)cache)[dst] = o[x];
        }
      }
    }
  }
  return 0;
}

/* ------------------------------------------------------------------ definitional fp64 */

/*  s_j = scale * <q, k_j> (* k_scale);  m = max(max_j s_j, sink);
 *  den = e^(sink-m) + sum_j e^(s_j-m);  out = sum_j e^(s_j-m) v_j (* v_scale) / den;
 *  lse = m + ln(den).  Two passes over the allowed keys, no online rescaling. */
int orc_attn_f64(const eid_attn_desc *d, const eid_attn_args *a, double *out64, double *lse64) {
  const int Hq = d->num_q_heads, Hkv = d->num_kv_heads, D = d->head_dim, B = d->block_size;
  const int G = Hq / Hkv;
  const uint16_t *q = (const uint16_t *)a->q;
  int rc = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < d->num_seqs; s++) {
    for (int h = 0; h < Hq; h++) {
      int row0, qlen;
      seq_rows(d, a, s, &row0, &qlen);
      const int L = a->seq_lens[s];
      const int kvh = h / G;
      const double ks = (d->kv_dtype == EID_KV_FP8_E4M3) ? (double)a->k_scale[kvh] : 1.0;
      const double vs = (d->kv_dtype == EID_KV_FP8_E4M3) ? (double)a->v_scale[kvh] : 1.0;
      const double sink = a->sinks ? (double)a->sinks[h] : -INFINITY;
      double *sc = (double *)malloc(sizeof(double) * (size_t)(L > 0 ? L : 1));
      for (int i = 0; i < qlen; i++) {
        const int p = L - qlen + i;
        double *o = out64 + ((size_t)(row0 + i) * Hq + h) * D;
        if (p < 0) { /* malformed: query before position 0 */
          rc = -1;
          for (int x = 0; x < D; x++) o[x] = NAN;
          continue;
        }
        const int lo = first_key(p, d->window);
        double qv[256];
        for (int x = 0; x < D; x++)
          qv[x] = (double)orc_bf16_to_f32(q[((size_t)(row0 + i) * Hq + h) * D + x]);
        double m = sink;
        for (int j = lo; j <= p; j++) {
          int64_t blk = a->block_table[(size_t)s * d->max_blocks_per_seq + j / B];
          size_t base = (((size_t)blk * B + j % B) * Hkv + kvh) * D;
          double acc = 0.0;
          for (int x = 0; x < D; x++) acc += qv[x] * kv_elem(a->k_cache, d->kv_dtype, base + x);
          sc[j] = acc * ks * (double)d->softmax_scale;
          if (sc[j] > m) m = sc[j];
        }
        double den = isinf(sink) ? 0.0 : exp(sink - m);
        for (int x = 0; x < D; x++) o[x] = 0.0;
        for (int j = lo; j <= p; j++) {
          double w = exp(sc[j] - m);
          den += w;
          int64_t blk = a->block_table[(size_t)s * d->max_blocks_per_seq + j / B];
          size_t base = (((size_t)blk * B + j % B) * Hkv + kvh) * D;
          for (int x = 0; x < D; x++) o[x] += w * kv_elem(a->v_cache, d->kv_dtype, base + x);
        }
        for (int x = 0; x < D; x++) o[x] = o[x] * vs / den;
        if (lse64) lse64[(size_t)(row0 + i) * Hq + h] = m + log(den);
      }
      free(sc);
    }
  }
  return rc;
}

/* ------------------------------------------------------------------ split-KV fp64 */

/* Partition c covers keys [kb + c*P, kb + (c+1)*P) intersected with the row's allowed set.
 * m_c = max s_j (-inf if none), l_c = sum e^(s_j-m_c), a_c = sum e^(s_j-m_c) v_j.  No sink. */
int orc_splitkv_partials_f64(const eid_attn_desc *d, const eid_attn_args *a, int32_t P,
                             int32_t nparts, double *part_ml, double *part_acc) {
  const int Hq = d->num_q_heads, Hkv = d->num_kv_heads, D = d->head_dim, B = d->block_size;
  const int G = Hq / Hkv;
  const uint16_t *q = (const uint16_t *)a->q;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < d->num_seqs; s++) {
    for (int h = 0; h < Hq; h++) {
      int row0, qlen;
      seq_rows(d, a, s, &row0, &qlen);
      const int L = a->seq_lens[s];
      const int kvh = h / G;
      const double ks = (d->kv_dtype == EID_KV_FP8_E4M3) ? (double)a->k_scale[kvh] : 1.0;
      const double vs = (d->kv_dtype == EID_KV_FP8_E4M3) ? (double)a->v_scale[kvh] : 1.0;
      const int kb = orc_kv_begin(L, qlen, d->window, B);
      double *sc = (double *)malloc(sizeof(double) * (size_t)P);
      for (int i = 0; i < qlen; i++) {
        const int p = L - qlen + i;
        const int lo = first_key(p, d->window);
        size_t row = (size_t)(row0 + i) * Hq + h;
        for (int c = 0; c < nparts; c++) {
          double *ml = part_ml + (row * nparts + c) * 2;
          double *acc = part_acc + (row * nparts + c) * D;
          int j0 = kb + c * P, j1 = j0 + P;
          if (j0 < lo) j0 = lo;
          if (j1 > p + 1) j1 = p + 1;
          ml[0] = -INFINITY;
          ml[1] = 0.0;
          for (int x = 0; x < D; x++) acc[x] = 0.0;
          if (j0 >= j1) continue;
          double m = -INFINITY;
          for (int j = j0; j < j1; j++) {
            int64_t blk = a->block_table[(size_t)s * d->max_blocks_per_seq + j / B];
            size_t base = (((size_t)blk * B + j % B) * Hkv + kvh) * D;
            double dot = 0.0;
            for (int x = 0; x < D; x++)
              dot += (double)orc_bf16_to_f32(q[row * D + x]) * kv_elem(a->k_cache, d->kv_dtype, base + x);
            sc[j - j0] = dot * ks * (double)d->softmax_scale;
            if (sc[j - j0] > m) m = sc[j - j0];
          }
          double l = 0.0;
          for (int j = j0; j < j1; j++) {
            double w = exp(sc[j - j0] - m);
            l += w;
            int64_t blk = a->block_table[(size_t)s * d->max_blocks_per_seq + j / B];
            size_t base = (((size_t)blk * B + j % B) * Hkv + kvh) * D;
            for (int x = 0; x < D; x++) acc[x] += w * kv_elem(a->v_cache, d->kv_dtype, base + x) * vs;
          }
          ml[0] = m;
          ml[1] = l;
        }
      }
      free(sc);
    }
  }
  return 0;
}

/* M = max(max_c m_c, sink); den = e^(sink-M) + sum_c l_c e^(m_c-M) (l_c = 0 skipped);
 * out = sum_c a_c e^(m_c-M) / den; lse = M + ln den.  Rows are (token, head) pairs,
 * head = row % Hq selects the sink. */
int orc_lse_merge_f64(int64_t T, int32_t Hq, int32_t nparts, int32_t D, const double *part_ml,
                      const double *part_acc, const float *sinks, double *out64, double *lse64) {
  for (int64_t r = 0; r < T * Hq; r++) {
    double sink = sinks ? (double)sinks[r % Hq] : -INFINITY;
    double M = sink;
    for (int c = 0; c < nparts; c++) {
      const double *ml = part_ml + ((size_t)r * nparts + c) * 2;
      if (ml[1] > 0.0 && ml[0] > M) M = ml[0];
    }
    double den = isinf(sink) ? 0.0 : exp(sink - M);
    double *o = out64 + (size_t)r * D;
    for (int x = 0; x < D; x++) o[x] = 0.0;
    for (int c = 0; c < nparts; c++) {
      const double *ml = part_ml + ((size_t)r * nparts + c) * 2;
      if (!(ml[1] > 0.0)) continue;
      double w = exp(ml[0] - M);
      den += ml[1] * w;
      const double *acc = part_acc + ((size_t)r * nparts + c) * D;
      for (int x = 0; x < D; x++) o[x] += acc[x] * w;
    }
    for (int x = 0; x < D; x++) o[x] /= den;
    if (lse64) lse64[r] = M + log(den);
  }
  return 0;
}

/* ------------------------------------------------------------------ CPU baseline (fp32) */

/* One pass over the pages of a sequence per (sequence, KV head): the G query heads that
 * share the KV head are advanced together with an online softmax in fp32; K/V rows are
 * widened once per page.  Output rounded RNE to bf16.  fp32 exp via expf. */
int orc_attn_bf16(const eid_attn_desc *d, const eid_attn_args *a, int num_threads) {
  const int Hq = d->num_q_heads, Hkv = d->num_kv_heads, D = d->head_dim, B = d->block_size;
  const int G = Hq / Hkv;
  if (D > 256 || G > 16) return -2;
  const uint16_t *q = (const uint16_t *)a->q;
  uint16_t *out = (uint16_t *)a->out;
#ifdef _OPENMP
  if (num_threads > 0) omp_set_num_threads(num_threads);
#endif
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < d->num_seqs; s++) {
    for (int kvh = 0; kvh < Hkv; kvh++) {
      int row0, qlen;
      seq_rows(d, a, s, &row0, &qlen);
      const int L = a->seq_lens[s];
      const float ks = (d->kv_dtype == EID_KV_FP8_E4M3) ? a->k_scale[kvh] : 1.0f;
      const float vs = (d->kv_dtype == EID_KV_FP8_E4M3) ? a->v_scale[kvh] : 1.0f;
      float kf[16 * 256], vf[16 * 256];
      for (int i = 0; i < qlen; i++) {
        const int p = L - qlen + i;
        const int lo = first_key(p, d->window);
        float qf[16][256], acc[16][256], m[16], l[16];
        for (int g = 0; g < G; g++) {
          int h = kvh * G + g;
          for (int x = 0; x < D; x++) {
            qf[g][x] = orc_bf16_to_f32(q[((size_t)(row0 + i) * Hq + h) * D + x]) * d->softmax_scale * ks;
            acc[g][x] = 0.f;
          }
          m[g] = -INFINITY;
          l[g] = 0.f;
        }
        for (int b0 = lo / B; b0 * B <= p; b0++) {
          int64_t blk = a->block_table[(size_t)s * d->max_blocks_per_seq + b0];
          int j0 = b0 * B < lo ? lo : b0 * B;
          int j1 = (b0 + 1) * B > p + 1 ? p + 1 : (b0 + 1) * B;
          for (int j = j0; j < j1; j++) {
            size_t base = (((size_t)blk * B + j % B) * Hkv + kvh) * D;
            for (int x = 0; x < D; x++) {
              kf[(j - j0) * D + x] = (float)kv_elem(a->k_cache, d->kv_dtype, base + x);
              vf[(j - j0) * D + x] = (float)kv_elem(a->v_cache, d->kv_dtype, base + x);
            }
          }
          for (int g = 0; g < G; g++) {
            float sc[64];
            float mb = m[g];
            for (int j = 0; j < j1 - j0; j++) {
              float dot = 0.f;
              for (int x = 0; x < D; x++) dot += qf[g][x] * kf[j * D + x];
              sc[j] = dot;
              if (dot > mb) mb = dot;
            }
            float corr = (m[g] == -INFINITY) ? 0.f : expf(m[g] - mb);
            l[g] *= corr;
            for (int x = 0; x < D; x++) acc[g][x] *= corr;
            for (int j = 0; j < j1 - j0; j++) {
              float w = expf(sc[j] - mb);
              l[g] += w;
              for (int x = 0; x < D; x++) acc[g][x] += w * vf[j * D + x];
            }
            m[g] = mb;
          }
        }
        for (int g = 0; g < G; g++) {
          int h = kvh * G + g;
          float sink = a->sinks ? a->sinks[h] : -INFINITY;
          float M = sink > m[g] ? sink : m[g];
          float w = expf(m[g] - M);
          float den = l[g] * w + (isinf(sink) ? 0.f : expf(sink - M));
          for (int x = 0; x < D; x++)
            out[((size_t)(row0 + i) * Hq + h) * D + x] = orc_f32_to_bf16(acc[g][x] * w * vs / den);
          if (a->lse) a->lse[(size_t)(row0 + i) * Hq + h] = M + logf(den);
        }
      }
    }
  }
  return 0;
}

/* ------------------------------------------------------------------ output projection */

/* out[t][n] = bf16(sum_k a[t][k] w[n][k] + bias[n] + residual[t][n]).  Every product of two
 * bf16 values is exact in double; the sum of K of them is accumulated in double (relative
 * error ~ K 2^-53, far below the bf16 grid). */
void orc_o_proj(const uint16_t *a, const uint16_t *w, const uint16_t *bias,
                const uint16_t *residual, uint16_t *out, double *exact64, int32_t T, int32_t N,
                int32_t K) {
#pragma omp parallel for schedule(static)
  for (int32_t t = 0; t < T; ++t) {
    for (int32_t n = 0; n < N; ++n) {
      const uint16_t *ar = a + (size_t)t * K, *wr = w + (size_t)n * K;
      double s = 0.0;
      for (int32_t k = 0; k < K; ++k) s += (double)orc_bf16_to_f32(ar[k]) * (double)orc_bf16_to_f32(wr[k]);
      if (bias) s += (double)orc_bf16_to_f32(bias[n]);
      if (residual) s += (double)orc_bf16_to_f32(residual[(size_t)t * N + n]);
      if (exact64) exact64[(size_t)t * N + n] = s;
      if (out) out[(size_t)t * N + n] = orc_f64_to_bf16(s);
    }
  }
}
