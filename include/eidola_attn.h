/*
 * eidola_attn.h — C ABI of the MI355X (gfx950) ragged-batch paged sink-attention path.
 *
 * Reference interface replaced: NONE EXISTS.  eidola-ai/eidola performs no inference
 * itself; its only seam towards an inference engine is an OpenAI-compatible HTTP
 * boundary (crates/eidola-server/src/backend.rs:87-108 `trait ChatBackend`,
 * crates/eidola-app-core/src/local_models.rs:1612-1626 engine spawn,
 * crates/eidola-app-core/src/lib.rs:6616-6623 HTTP POST).  No tensor, pointer or shape
 * crosses it.  Every entry point below is therefore defined by this library; each
 * comment says which stage of the path it is and which engine-side call site would
 * bind it.
 *
 * Conventions
 *  - All tensor pointers are DEVICE pointers owned by the caller; the library allocates
 *    no device memory.  State it keeps: a thread-local error string; per process, cached
 *    read-only facts about the device (CU count, the kernels' register and LDS footprints),
 *    queried on first use; per calling thread and device, one helper stream and two events,
 *    created by the thread's first mixed prefill + decode call of eid_attn_varlen and
 *    destroyed when the thread ends; per device, the static workspace of
 *    eid_attn_decode_noalloc; per process, what the eid_debug_* measurement aids were last
 *    given (a buffer pointer, two events; all null unless a measurement set them).
 *  - All work is enqueued asynchronously on the caller's `hipStream_t`
 *    (passed as `void *`; NULL = the default stream).
 *  - Every function returns an `eid_status` (0 = OK, negative = error) and never
 *    throws or aborts.  Argument validation needs no GPU: invalid-argument paths can be
 *    exercised on a host without one.  Planning (eid_workspace_bytes, eid_partition_size)
 *    asks the runtime for the device's CU count; without a device it assumes 256, the
 *    MI355X's, so the sizes computed on a GPU-less host are the ones the GPU box uses.
 *  - HIP graphs: every entry point may be called on a capturing stream (kernels and event
 *    nodes only).  A captured call serves later replays with other device-side seq_lens /
 *    block_table contents as long as the descriptor's max_kv_len and sum_kv_len bound them.
 *    The optional HOST copies of those arrays are ignored while the stream is capturing: a
 *    plan made from them would be frozen into the graph.
 *
 * Geometry supported by this version: head_dim 64, block_size 16,
 * num_q_heads = 8 * num_kv_heads (GQA 8:1), bf16 Q/out, bf16 or fp8-e4m3fn KV.
 *
 * Tensor layouts (row-major, innermost last)
 *   q, out            [num_q_tokens, num_q_heads, 64]  bf16   ragged by cu_seqlens_q
 *   k_new, v_new      [num_tokens,   num_kv_heads, 64] bf16
 *   k_cache, v_cache  [num_blocks, 16, num_kv_heads, 64]  bf16 or fp8-e4m3fn
 *   slot_mapping      [num_tokens] int64   slot = block*16 + offset, -1 = skip
 *   block_table       [num_seqs, max_blocks_per_seq] int32   entries past a sequence's last page
 *                     are never needed; ids are clamped to [0, num_blocks) and lengths to the
 *                     row before use, so junk there cannot make a kernel leave the caches
 *   cu_seqlens_q      [num_seqs + 1] int32
 *   seq_lens          [num_seqs] int32   KV length AFTER this step's append
 *   sinks             [num_q_heads] fp32 (NULL = no sink, i.e. -inf)
 *   k_scale, v_scale  [num_kv_heads] fp32 (fp8 only)
 *   lse               [num_q_tokens, num_q_heads] fp32 (optional) = m + ln(denominator).
 *                     Asking for it selects the prefill kernel that keeps the softmax factor
 *                     out of its bf16 Q operands (a few per cent slower; `out` differs from
 *                     the call without lse by at most a bf16 ulp on prefill rows).
 */
#ifndef EIDOLA_ATTN_H
#define EIDOLA_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EID_VERSION_MAJOR 0
#define EID_VERSION_MINOR 1

typedef enum {
  EID_OK = 0,
  EID_ERR_INVALID_ARG = -1, /* null pointer, bad shape, misalignment, bad struct_size */
  EID_ERR_UNSUPPORTED = -2, /* geometry or dtype outside what this version builds    */
  EID_ERR_WORKSPACE = -3,   /* workspace NULL or smaller than eid_workspace_bytes()  */
  EID_ERR_HIP = -4,         /* a HIP runtime call or kernel launch failed            */
  EID_ERR_NO_BLOCKS = -5    /* eidola_sched.h: the KV pool cannot hold the request   */
} eid_status;

typedef enum { EID_KV_BF16 = 0, EID_KV_FP8_E4M3 = 1 } eid_kv_dtype;

/* Shapes and scalars.  Plain data; `struct_size` must be sizeof(eid_attn_desc). */
typedef struct eid_attn_desc {
  uint32_t struct_size;
  int32_t num_seqs;
  int32_t num_q_tokens;       /* total rows of q / out                                   */
  int32_t max_q_len;          /* max over sequences of cu_seqlens_q[s+1]-cu_seqlens_q[s] */
  int32_t max_kv_len;         /* max over sequences of seq_lens[s]                       */
  int32_t num_q_heads;        /* 64 */
  int32_t num_kv_heads;       /* 8  */
  int32_t head_dim;           /* 64 */
  int32_t block_size;         /* 16 */
  int32_t max_blocks_per_seq; /* row stride of block_table                               */
  int64_t num_blocks;         /* blocks in each of k_cache / v_cache                     */
  float softmax_scale;        /* 1/sqrt(head_dim) normally                               */
  int32_t window;             /* 0 = full causal; W>0: row at position p sees p-W+1..p   */
  int32_t kv_dtype;           /* eid_kv_dtype                                            */
  int32_t partition_size;     /* split-KV partition in tokens: a multiple of 64 in
                                 [64, 4096], or 0 = the library cuts the batch itself, into
                                 equal ranges of 64-key chunks (>= 256 keys each).  A non-zero
                                 value is the grid on which a sequence may be cut.  Long
                                 launches are cut into equal contiguous ranges of partitions,
                                 one per workgroup; a workgroup that holds several consecutive
                                 partitions of a sequence merges them in registers and stores
                                 one partial for the whole piece (stores trickling into the
                                 stream of loads are dear on this machine).  Results do not
                                 depend on it beyond fp32 round-off.                      */
  int64_t sum_kv_len;         /* optional launch-sizing hint: any value >= the sum of
                                 seq_lens[s] over the batch, or 0 = not known.  An engine's
                                 scheduler holds seq_lens on the host, so the sum is free;
                                 with it the split-KV grid is sized to the work instead of
                                 to num_seqs * max_kv_len.  A value below the true sum is a
                                 caller error the library cannot detect (work is dropped). */
} eid_attn_desc;

/* Device pointers, all caller-owned. */
typedef struct eid_attn_args {
  const void *q;
  void *out;
  float *lse; /* may be NULL */
  const void *k_cache;
  const void *v_cache;
  const int32_t *block_table;
  const int32_t *cu_seqlens_q; /* may be NULL for eid_attn_decode (q_len == 1 for all) */
  const int32_t *seq_lens;
  const float *sinks;   /* may be NULL */
  const float *k_scale; /* fp8 only */
  const float *v_scale; /* fp8 only */
  void *workspace;      /* >= eid_workspace_bytes(desc), 256-byte aligned */
  size_t workspace_bytes;
  void *split_done_event; /* optional hipEvent_t (NULL = none), for profiling: recorded on the
                             stream right after the split-KV launch of the q_len <= 2 class,
                             i.e. before its merge, so that a caller who records an event of
                             his own before the call can time that kernel by itself */
  const void *k_new;    /* eid_attn_decode only, optional (both or neither): [num_seqs, Hkv, 64] */
  const void *v_new;    /* bf16 rows of every sequence's newest token (position seq_lens[s]-1),
                           NOT yet in the cache.  The call then writes them into k_cache /
                           v_cache itself (same bits as eid_kv_write to slot
                           block_table[s][pos/16]*16 + pos%16) and attends to them from
                           registers: the step needs no separate eid_kv_write launch.
                           k_cache / v_cache are written in that case. */
  const int32_t *seq_lens_host;     /* optional HOST copies of seq_lens [num_seqs] and */
  const int32_t *cu_seqlens_q_host; /* cu_seqlens_q [num_seqs + 1] (the latter is needed by
                           eid_attn_varlen only), read before the call returns.  An engine's
                           scheduler builds these arrays on the host anyway; with them the
                           library plans the launches itself (partition size, exact grids,
                           which kernels have work at all) instead of leaving that to every
                           workgroup of the kernels.  They must equal the device arrays
                           (EID_DEBUG=1 in the environment makes the call verify that, with a
                           device synchronisation); results do not depend on whether they are
                           given.  Ignored on a capturing stream (see "HIP graphs" above). */
  const int32_t *block_table_host;  /* optional HOST copy of block_table (same shape), used by
                           eid_attn_decode together with seq_lens_host: the page ids of every
                           work item's first chunk then travel with the launch instead of
                           being fetched by the workgroup before its first K/V load */
} eid_attn_args;

/*
 * Stage K1 — slot-mapped KV-cache write ("reshape and cache").
 * cache_flat[slot_mapping[t], h, :] = f(k_new[t, h, :]) for every t with slot >= 0.
 * bf16: bit copy.  fp8: RNE_e4m3fn(clamp(fp32(x) / scale[h], -448, 448)), NaN -> 0x7F.
 * Only desc->num_kv_heads, head_dim, block_size, num_blocks, kv_dtype are read.
 * Reference counterpart: none.  Engine call site: once per layer per step, after the
 * QKV projection and before attention, on the same stream.
 */
int32_t eid_kv_write(const eid_attn_desc *desc, const void *k_new, const void *v_new,
                     void *k_cache, void *v_cache, const int64_t *slot_mapping,
                     int32_t num_tokens, const float *k_scale, const float *v_scale,
                     void *hip_stream);

/*
 * The step in front of K1, fused with it: rotary embedding of q and k (half-split pairing,
 * dim i with dim i + 32), split of the projection output into q / k / v, and the slot-mapped
 * KV write, in one pass over the new tokens.
 *   qkv        [num_tokens, (Hq + 2 Hkv) * 64] bf16: per token the q heads, then the k heads,
 *              then the v heads
 *   positions  [num_tokens] int32, absolute position of each token; values outside
 *              [0, max_pos) are clamped into the table
 *   cos_sin    [max_pos, 64] fp32: per position 32 cosines then 32 sines, already multiplied
 *              by whatever attention-temperature factor the model's RoPE scaling prescribes
 *   q_out      [num_tokens, Hq, 64] bf16
 * Arithmetic (fixed, so that results are reproducible bit for bit): with x1 = x[i],
 * x2 = x[i + 32] in fp32, o[i] = fma(-x2, sin_i, x1 * cos_i), o[i + 32] = fma(x1, sin_i,
 * x2 * cos_i), each rounded to bf16 nearest-even; the rotated k row and the v row are then
 * stored exactly as eid_kv_write stores a bf16 row (fp8: quantised from the bf16 value).
 * Tokens with slot -1 still produce q_out.  Reference counterpart: none.  Engine call site:
 * once per layer per step after the QKV projection, instead of a RoPE kernel + eid_kv_write.
 */
int32_t eid_rope_kv_write(const eid_attn_desc *desc, const void *qkv, const int32_t *positions,
                          const float *cos_sin, int32_t max_pos, void *q_out, void *k_cache,
                          void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                          const float *k_scale, const float *v_scale, void *hip_stream);

/*
 * Stages K2+K4 — decode attention: every sequence contributes exactly one query row
 * (num_q_tokens == num_seqs, max_q_len == 1).  Split-KV over partitions of
 * `partition_size` tokens with the per-head sink folded into the denominator once, in
 * the merge.  Reference counterpart: none.  Engine call site: per layer per decode step.
 */
int32_t eid_attn_decode(const eid_attn_desc *desc, const eid_attn_args *args,
                        void *hip_stream);

/*
 * eid_attn_decode for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has NO counterpart in
 * the reference (nor does anything else here) and exists for those callers only.
 * Same arguments, same kernels and bit-identical results as eid_attn_decode, except that
 * args->workspace / args->workspace_bytes are ignored: the split-KV partials go to a static
 * device array of EID_STATIC_WORKSPACE_BYTES that the library holds on every GPU it runs on
 * until the process ends.  The call allocates nothing, on the device or on the host (no
 * hipMalloc / hipFree, no allocating library routine); the first call on a device looks the
 * array's address up once.  A batch with eid_workspace_bytes(desc) above that size is
 * rejected with EID_ERR_WORKSPACE (use eid_attn_decode with a workspace of your own); for
 * batches of more than 1,024 sequences the host copies of the lengths are not used for
 * planning.  All calls on one GPU share the one array: calls that overlap in time on the
 * same GPU (two streams, two threads, two graphs in flight) race on it; serialise them, or
 * give the others eid_attn_decode with their own workspace.  Nothing in the array has to
 * start from a particular value, so it is never cleared.  With EID_DEBUG=1 in the environment
 * the call remembers, per GPU, the stream of the last call and an event behind it, and returns
 * EID_ERR_INVALID_ARG when a call arrives on another stream while that event is pending (the
 * checking mode creates one event per GPU: it does allocate).
 */
#define EID_STATIC_WORKSPACE_BYTES (32u << 20)
int32_t eid_attn_decode_noalloc(const eid_attn_desc *desc, const eid_attn_args *args,
                                void *hip_stream);

/*
 * Stages K2/K3+K4 — ragged attention in cu_seqlens layout: chunked prefill, speculative
 * verify and mixed prefill+decode batches.  Query row i of sequence s sits at absolute
 * position seq_lens[s] - q_len_s + i and sees keys 0..position (clipped by `window`).
 * Sequences with q_len <= 6 (<= 8 when desc->max_q_len <= 8; <= 16 when desc->max_q_len <= 16,
 * num_kv_heads % 8 == 0 and num_seqs * num_kv_heads <= 448; <= 32 when desc->max_q_len <= 32 and
 * num_seqs * num_kv_heads <= 64) run on the bandwidth-bound split-KV kernel; longer chunks
 * run on the bf16-MFMA tile kernel.  Reference counterpart: none.
 */
int32_t eid_attn_varlen(const eid_attn_desc *desc, const eid_attn_args *args,
                        void *hip_stream);

/*
 * Stage K4 alone — merge the split-KV partials found in args->workspace (as laid out by
 * the split-KV kernel for this desc) into args->out / args->lse.  Exposed for tests.
 * Serves one class of sequences per call, as the split-KV launches do: q_len <= 2 when
 * desc->max_q_len <= 2, otherwise q_len 3..6 (3..8, 3..16 or 3..32 under the conditions above).  Sequences with a single partition are left
 * alone (the split-KV kernel writes their output itself).  With desc->partition_size == 0
 * the partition is the one the last eid_attn_decode / eid_attn_varlen call on this
 * workspace recorded in its header, so such a call must have preceded.
 * Workspace layout, with R = min(max_q_len, 6) (min(max_q_len, 8), 16 or 32 under the conditions above) and N = partitions per sequence (max; one more
 * with partition_size == 0, whose ranges are cut anywhere in a sequence):
 *   256 bytes                         launch plan (written by the library)
 *   int32 parts [num_seqs]            (only when N > 1, padded to 256 bytes) pieces per sequence
 *                                     as the last even split left them
 *   float ml [num_seqs*R][N][Hq][2]   m (natural-log units, -inf if empty) and
 *                                     l = sum of e^(s-m) over the partition's keys
 *   half  o  [num_seqs*R][N][Hq][64]  the partition's own output sum e^(s-m) v / l (fp16,
 *                                     saturated at +-65504), at the next 256-byte boundary
 * Range of values: a partial output is a convex combination of value rows (times v_scale), so
 * sequences of several partitions are exact to fp16 while |v| <= 65504; larger entries (bf16
 * can hold them) saturate there, in those sequences only.
 * (heads innermost: the 64 heads of one (row, partition) cell form one contiguous block,
 * which a split-KV workgroup writes with full-width stores)
 * Behind these, when the batch holds prefill chunks whose query tiles cannot fill the device
 * by themselves (few new tokens behind a long context), the same two arrays once more for the
 * prefill rows, [num_q_tokens][K] cells with K <= 8 key-range parts per query tile; they are
 * merged inside the call.  eid_workspace_bytes() accounts for all of it.
 */
int32_t eid_lse_merge(const eid_attn_desc *desc, const eid_attn_args *args,
                      void *hip_stream);

/*
 * The step behind the path: output projection with bias and residual epilogue,
 *   out[t, n] = bf16( sum_k attn_out[t, k] * weight[n, k] + bias[n] + residual[t, n] ),
 * products and sums in fp32, one rounding to bf16 (nearest-even) at the end.
 *   attn_out  [num_tokens, in_features] bf16: the `out` of eid_attn_decode / eid_attn_varlen
 *             as it stands ([num_q_tokens, Hq, 64], in_features = Hq * 64, index
 *             head * 64 + dim): token-major rows are the K-contiguous operand the matrix
 *             units want, so no head-major variant of the attention output exists
 *   weight    [out_features, in_features] bf16, in_features contiguous (the usual order of
 *             a linear layer's weight)
 *   bias      [out_features] bf16 or NULL
 *   residual  [num_tokens, out_features] bf16 or NULL; may be the same buffer as `out`
 *   out       [num_tokens, out_features] bf16
 * in_features must be a multiple of 64, out_features a multiple of 16; all pointers 16-byte
 * aligned.  Up to 64 tokens the weight is streamed once (HBM-bound), beyond that a tiled
 * matrix-core kernel runs.  The order of the fp32 additions differs between the two and from
 * a sequential sum; results agree with an exactly rounded result to within fp32 summation
 * error before the bf16 rounding.  Reference counterpart: none.  Engine call site: per layer
 * per step, right after attention, on the same stream.
 */
int32_t eid_o_proj(const void *attn_out, const void *weight, const void *bias,
                   const void *residual, void *out, int32_t num_tokens, int32_t out_features,
                   int32_t in_features, void *hip_stream);

/*
 * QKV projection and eid_rope_kv_write in ONE launch, for decode-sized batches
 * (num_tokens <= 64; EID_ERR_UNSUPPORTED beyond: use eid_o_proj, then eid_rope_kv_write):
 *   qkv = hidden @ weight^T + bias        hidden [num_tokens, in_features] bf16,
 *                                         weight [(Hq + 2 Hkv) * 64, in_features] bf16,
 *                                         bias   [(Hq + 2 Hkv) * 64] bf16 or NULL
 * followed by exactly what eid_rope_kv_write does with that qkv (rotation of the q and k
 * heads by positions[t], q rows to q_out, k and v rows into their cache slots), with the
 * same arithmetic on the same bf16-rounded projection outputs: q_out and the caches come
 * out bit-identical to the two calls, and the [num_tokens, (Hq + 2 Hkv) * 64] intermediate
 * is never written.  in_features % 64 == 0.  Other arguments as eid_rope_kv_write.
 * Reference counterpart: none.
 */
int32_t eid_qkv_rope_kv_write(const eid_attn_desc *desc, const void *hidden, const void *weight,
                              const void *bias, int32_t in_features, const int32_t *positions,
                              const float *cos_sin, int32_t max_pos, void *q_out, void *k_cache,
                              void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                              const float *k_scale, const float *v_scale, void *hip_stream);

/* Bytes of workspace eid_attn_decode / eid_attn_varlen / eid_lse_merge need for desc.
 * Returns 0 for an invalid desc. */
size_t eid_workspace_bytes(const eid_attn_desc *desc);

/* The partition size (tokens) the workspace is planned with: desc->partition_size; when that
 * is 0, the lower bound 256 of the kernels' run-time choice, or, for a batch with at least
 * one sequence per compute unit whose longest span fits one partition (2,048 tokens), that
 * span rounded up to 64: every sequence is then one work item and no partials are written;
 * or, for a batch so small that every 64-token chunk gets a wavefront of its own at once
 * (one workgroup of eight per 512 tokens and KV head, all resident together), 512. */
int32_t eid_partition_size(const eid_attn_desc *desc);

/* Thread-local description of the last error on this thread; "" if none. */
const char *eid_last_error(void);

/* (major << 16) | minor */
uint32_t eid_version(void);

#ifdef __cplusplus
}
#endif
#endif /* EIDOLA_ATTN_H */
