/*
 * eid_oracle.h — CPU oracle for the paged sink-attention path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the product library links or calls this; only tests/, the smoke check and
 * the benchmark's cpu_baseline leg load liboracle.so.
 *
 * Reference file followed: none exists.  eidola-ai/eidola holds no attention, KV-cache or
 * kernel code (its inference is proxied: docs/server.md:102-109,
 * crates/eidola-server/src/backend.rs:421-478), so every function here restates the
 * mathematical definition of the path, and parity with "the reference" is UNPINNED by
 * construction.  What pins these functions instead: closed forms of softmax-with-sink,
 * torch's scaled_dot_product_attention for the sink = -inf special case, an independent
 * numpy restatement, brute force on tiny inputs, exhaustive fp8 round trips against an
 * independently written encoder, and paging/partition invariances (see tests/).
 *
 * All pointers are HOST pointers; layouts and the descriptor are those of
 * include/eidola_attn.h.
 */
#ifndef EID_ORACLE_H
#define EID_ORACLE_H
#include <stdint.h>
#include <stddef.h>
#include "../include/eidola_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar conversions ---- */
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);                 /* round-to-nearest-even, NaN -> quiet NaN */
uint8_t orc_fp8_e4m3_encode(float x);              /* RNE, saturate to +-448, NaN -> 0x7F     */
float orc_fp8_e4m3_decode(uint8_t b);              /* exact; 0x7F / 0xFF -> NaN               */

/* ---- the path ---- */
/* K1: same contract as eid_kv_write. Returns 0, or -1 on an out-of-range slot. */
int orc_kv_write(const eid_attn_desc *d, const uint16_t *k_new, const uint16_t *v_new,
                 void *k_cache, void *v_cache, const int64_t *slot_mapping,
                 int32_t num_tokens, const float *k_scale, const float *v_scale);

/* Fused RoPE + QKV split + KV write: same contract as eid_rope_kv_write.  Returns 0, or -1
 * on an out-of-range slot. */
int orc_rope_kv_write(const eid_attn_desc *d, const uint16_t *qkv, const int32_t *positions,
                      const float *cos_sin, int32_t max_pos, uint16_t *q_out, void *k_cache,
                      void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                      const float *k_scale, const float *v_scale);

/* Output projection with bias and residual: same contract as eid_o_proj.
 * exact64 (may be NULL) receives the unrounded values [T, N]: the fp64 sum of the exact
 * bf16 x bf16 products, plus bias, plus residual; out (may be NULL) receives them rounded to
 * bf16 once, nearest-even, straight from the double (no detour through fp32). */
void orc_o_proj(const uint16_t *a, const uint16_t *w, const uint16_t *bias,
                const uint16_t *residual, uint16_t *out, double *exact64, int32_t T, int32_t N,
                int32_t K);
uint16_t orc_f64_to_bf16(double x);                /* round-to-nearest-even, NaN -> quiet NaN */

/* Definitional attention in fp64 from the stored bf16/fp8 bits.
 * out64: [T, Hq, D] doubles; lse64: [T, Hq] doubles or NULL.
 * cu_seqlens_q may be NULL (then q_len = 1 for every sequence). */
int orc_attn_f64(const eid_attn_desc *d, const eid_attn_args *host, double *out64,
                 double *lse64);

/* Split-KV restatement in fp64: partials per (row, head, partition) WITHOUT the sink
 * (m = -inf, l = 0, acc = 0 for an empty partition), then the merge WITH the sink.
 * part_ml: [T, Hq, nparts, 2]; part_acc: [T, Hq, nparts, D].  Partition c of a sequence
 * covers keys [kv_begin + c*P, kv_begin + (c+1)*P), kv_begin = orc_kv_begin(...). */
int orc_splitkv_partials_f64(const eid_attn_desc *d, const eid_attn_args *host, int32_t P,
                             int32_t nparts, double *part_ml, double *part_acc);
/* rows are (token, head) pairs; head = row % Hq selects sinks[head] (sinks may be NULL). */
int orc_lse_merge_f64(int64_t T, int32_t Hq, int32_t nparts, int32_t D, const double *part_ml,
                      const double *part_acc, const float *sinks, double *out64, double *lse64);
/* First key any query row of the sequence can see, rounded down to a block boundary. */
int32_t orc_kv_begin(int32_t seq_len, int32_t q_len, int32_t window, int32_t block_size);

/* CPU production-style path: fp32 accumulation, online softmax over 16-token pages,
 * OpenMP over (sequence, KV head), bf16 output.  This is the timed CPU baseline. */
int orc_attn_bf16(const eid_attn_desc *d, const eid_attn_args *host, int num_threads);

#ifdef __cplusplus
}
#endif
#endif
