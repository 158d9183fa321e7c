/*
 * eidola_sched.h — C ABI of the paged-KV block allocator and batch-metadata builder: the
 * host-side caller of the attention path in eidola_attn.h.
 *
 * Reference interface replaced: NONE EXISTS.  eidola-ai/eidola keeps no KV cache (its local
 * engine is an external `llama-server -c 8192` process,
 * crates/eidola-app-core/src/local_models.rs:1612-1626, and the nearest thing to cache
 * accounting is a RAM-budget estimate, local_models.rs:61 and :588).  An engine that hosts
 * the attention kernels needs exactly this component to turn a continuous-batching schedule
 * ("these sequences advance by so many tokens this step") into the arrays the kernels take:
 * block_table, slot_mapping, cu_seqlens_q, seq_lens, positions, and the host-side scalars
 * max_q_len, max_kv_len and sum_kv_len of eid_attn_desc.
 *
 * Everything here is HOST code: no HIP call, no device memory.  The arrays are written into
 * caller-owned host buffers (pinned, if the caller wants to copy them asynchronously).
 * A scheduler object is not thread-safe; use one per engine thread or lock around it.
 *
 * Blocks are block_size (16) tokens.  A sequence owns a list of physical blocks; the last one
 * may be partly filled.  Full blocks are immutable and, with prefix reuse enabled, indexed by
 * a chained hash of their token ids so that a new sequence with the same prefix maps to the
 * same physical blocks (reference counted) and only computes the rest of its prompt.  Freed
 * blocks keep their hash until the allocator hands them out again (least recently freed
 * first), so a prefix can be hit after its last owner has gone.
 */
#ifndef EIDOLA_SCHED_H
#define EIDOLA_SCHED_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct eid_sched eid_sched; /* opaque */

typedef struct eid_sched_config {
  uint32_t struct_size;       /* sizeof(eid_sched_config) */
  int32_t block_size;         /* tokens per block: 16 */
  int64_t num_blocks;         /* blocks in each of k_cache / v_cache */
  int32_t max_blocks_per_seq; /* row stride of the block tables this scheduler fills */
  int32_t prefix_reuse;       /* 0 = off, 1 = share full blocks between equal prefixes */
} eid_sched_config;

/* What one built batch looks like; the scalar fields go straight into eid_attn_desc. */
typedef struct eid_batch_info {
  int32_t num_seqs;
  int32_t num_q_tokens; /* sum of q_lens */
  int32_t max_q_len;
  int32_t max_kv_len;
  int64_t sum_kv_len;   /* sum of seq_lens: the launch-sizing hint of eid_attn_desc */
} eid_batch_info;

/* Status codes are those of eidola_attn.h: EID_OK, EID_ERR_INVALID_ARG, and
 * EID_ERR_NO_BLOCKS (-5: the pool cannot hold the request; nothing was changed).
 * eid_last_error() describes the failure. */

int32_t eid_sched_create(const eid_sched_config *cfg, eid_sched **out);
void eid_sched_destroy(eid_sched *s);

/* Registers a sequence.  With prefix reuse, `prompt` (n token ids) is matched block by block
 * against the index; the matched blocks become the head of the sequence's block list and
 * their tokens count as already present in the cache.  At least one prompt token is always
 * left to compute.  Without prefix reuse (or prompt == NULL) the sequence starts empty.
 * Returns the number of cached tokens in *cached_tokens (may be NULL). */
int32_t eid_sched_add_seq(eid_sched *s, int64_t seq_id, const int32_t *prompt, int32_t n,
                          int32_t *cached_tokens);

/* Drops a sequence: its blocks lose one reference each; unreferenced blocks join the free
 * list (keeping their hash, see above). */
int32_t eid_sched_free_seq(eid_sched *s, int64_t seq_id);

/* Tokens currently in the cache for seq_id, or -1 if unknown. */
int32_t eid_sched_seq_len(const eid_sched *s, int64_t seq_id);
/* Blocks no sequence references (allocatable). */
int64_t eid_sched_free_blocks(const eid_sched *s);
/* Reference count of a physical block (0 = free), -1 if out of range.  For tests. */
int32_t eid_sched_block_refs(const eid_sched *s, int64_t block);

/*
 * Builds the metadata of one step.  Sequence i = seq_ids[i] advances by q_lens[i] >= 1 new
 * tokens (prefill chunk, verify rows, or 1 for decode); their KV slots are reserved here.
 * All-or-nothing: if the pool cannot hold every new token the call fails with EID_ERR_NO_BLOCKS and no
 * sequence has changed.
 *
 *   new_tokens     [sum q_lens] token ids of the new tokens, sequence after sequence; needed
 *                  to index blocks that become full (prefix reuse); may be NULL otherwise
 *   block_table    [num_seqs, max_blocks_per_seq] int32, filled up to each sequence's blocks
 *                  (the rest of a row is left untouched)
 *   slot_mapping   [sum q_lens] int64   slot = block * block_size + offset of each new token
 *   cu_seqlens_q   [num_seqs + 1] int32
 *   seq_lens       [num_seqs] int32     KV length after this step's append
 *   positions      [sum q_lens] int32   absolute position of each new token (for RoPE); may
 *                  be NULL
 *   info           scalars of the batch
 */
int32_t eid_sched_build_batch(eid_sched *s, const int64_t *seq_ids, const int32_t *q_lens,
                              int32_t num_seqs, const int32_t *new_tokens,
                              int32_t *block_table, int64_t *slot_mapping,
                              int32_t *cu_seqlens_q, int32_t *seq_lens, int32_t *positions,
                              eid_batch_info *info);

#ifdef __cplusplus
}
#endif
#endif /* EIDOLA_SCHED_H */
