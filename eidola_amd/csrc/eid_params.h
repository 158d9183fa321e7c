// Host/device launch descriptors of the attention kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

namespace eid {

constexpr int kHeadDim = 64;
constexpr int kBlock = 16;        // tokens per KV page
constexpr int kGroup = 8;         // query heads per KV head
constexpr int kShortQMax = 6;     // q_len handled by the split-KV kernel (6*8 = 48 rows = 3 tiles)
constexpr int kShortQMaxWide = 8; // ... when no sequence of the batch has more than 8 rows: four tiles
constexpr int kShortQMaxRows = 16; // ... or more than 16: two waves of four tiles share a KV head
constexpr int kShortQMaxRows4 = 32; // ... or 32: four waves per KV head
constexpr int kRows4MaxGroups = 64;  // num_seqs * Hkv up to which 17..32 rows take four waves per KV head
constexpr int kRowsMaxGroups = 448; // ... the latter only for num_seqs * Hkv up to this (see short_q_max)
constexpr int kChunk = 64;        // tokens a wave consumes per iteration of the split-KV loop
constexpr int kDynPartitionMin = 256;   // lower bound (and workspace sizing) of the dynamic partition
constexpr int kDynPartitionCap = 2048;  // a workgroup streams serially: keep its share bounded
constexpr int kDynPartitionFloor = 512; // smallest partition when the batch needs several fills
constexpr int kShortSpanMax = 512;      // keys one workgroup of the short-span kernel covers
constexpr int kPlanBytes = 256;         // head of the workspace: two {partition, items} slots
// Size of the library's own split-KV workspace (a static device array, one copy per GPU),
// which the decode entry point that allocates nothing uses in place of a caller's workspace.
constexpr size_t kStaticScratchBytes = 32u << 20;
constexpr int kStackPlanSeqs = 1024;    // sequences the host plans for without heap storage
constexpr int kEvenMinChunks = kDynPartitionMin / kChunk;  // chunks per workgroup of an even split, at least
constexpr int kEvenFlag = 1 << 29;      // plan slot of an even split that stored pieces: flag | quota

struct AttnParams {
  const uint16_t *q;
  uint16_t *out;
  float *lse;
  const uint8_t *k_cache;
  const uint8_t *v_cache;
  const uint16_t *k_new;  // decode only, may be NULL: [num_seqs, Hkv, 64] bf16 rows of the newest
  const uint16_t *v_new;  // token of every sequence, written into the caches by this launch
  const int32_t *block_table;
  const int32_t *cu_seqlens_q;  // may be null: q_len == 1 everywhere
  const int32_t *seq_lens;
  const float *sinks;    // may be null
  const float *k_scale;  // fp8 only
  const float *v_scale;  // fp8 only
  const int32_t *plan;   // {partition, number of items} written by the plan kernel, or null
  int32_t *plan_slot;    // where this launch's split-KV kernel records its partition for the merge
  int32_t *seq_parts;    // [num_seqs] pieces per sequence, written by an even split for its merge
                         // (the pieces have no common size)
  int32_t even_wgs;      // workgroups of an even split (its grid)
  int32_t mixed_wgs;     // host-side: cap on even_wgs for the split-KV rows of a mixed batch, 0 = none
  int32_t store_every_partition;  // even split with the caller's partition: a partial per partition
                         // instead of one per piece (measurement aid, EID_STORE_EVERY_PARTITION)
  float *ws_ml;          // [num_seqs*ws_rows][nparts_max][Hq][2]  (m natural-log units, l)
  _Float16 *ws_acc;      // [num_seqs*ws_rows][nparts_max][Hq][64] partition output, normalised
  int32_t target_items_lo; // workgroups at one per CU (<= target_items)
  long long sum_kv_len;  // host's upper bound on the sum of seq_lens, 0 = unknown
  int32_t num_seqs, num_q_heads, num_kv_heads, max_blocks_per_seq;
  int32_t last_block;    // num_blocks - 1: every page id is clamped to [0, last_block] before
                         // use, so a stale or wrong table entry reads a wrong page, never
                         // memory outside the caches
  int32_t window, partition, nparts_max, ws_rows;
  int32_t qlen_lo, qlen_hi;  // this launch serves sequences with qlen_lo <= q_len <= qlen_hi
  int32_t dynamic_partition; // 1: kernels derive the partition from the batch (>= partition)
  int32_t target_items;      // workgroups the device holds at once (dynamic partition only)
  int32_t pf_splits;         // prefill kernel: every query tile's key range is split into this
                             // many parts (1 = none); parts write partials to pf_ml / pf_acc
  float *pf_ml;              // [num_q_tokens][pf_splits][Hq][2]   (m natural-log units, l)
  _Float16 *pf_acc;          // [num_q_tokens][pf_splits][Hq][64]  part output, normalised
  int32_t num_q_tokens;
  int32_t fp8_pair;          // host-side launch flag: 1 = every sequence has one query row, fp8 cache,
                             // eight KV heads: the split-KV launch may give each wave two KV heads
  int32_t share_cus;         // host-side launch flag: 1 = hold the split-KV kernel to one
                             // workgroup per CU (a prefill launch runs beside it)
  int32_t dma;               // host-side launch flag: 1 = bf16 cache and no prefill launch beside: the
                             // split-KV kernels stream their chunks by direct global -> LDS loads
  int32_t dma_pair;          // host-side launch flag: fp8 head pairs of an even split stream through LDS too
  int32_t dma_fp8;           // host-side launch flag: so do verify rows over an fp8 cache (one head per wave)
  long long exact_items;     // host-side: the launch's exact number of work items when the host
                             // has the sequence lengths, 0 = not known (a bound is launched)
  float softmax_scale;
  // Measurement aid, null in normal use: wave w of workgroup b of the prefill kernel
  // stores {start, end} (100 MHz wall-clock ticks), {hardware id, XCC id} and up to
  // four stamps in between at timeline[(b * waves + w) * 8 ..]; see set_timeline().
  unsigned long long *timeline;
};

// Work items of a decode launch listed by the host (it has the sequence lengths): entry =
// seq | part << 16 | seq_len << 32.  Passed by value as a kernel argument, so a workgroup has
// its item after one scalar load instead of a scan of seq_lens.
constexpr int kItemTableMax = 384;
struct ItemTable {
  int32_t n;
  int32_t has_blk;  // blk[] holds the page ids of every item's first four pages
  unsigned long long e[kItemTableMax];
  int32_t blk[kItemTableMax][4];
};

// Start of every workgroup's range in an even split (see splitkv_even_kernel), listed by the
// host when it has the sequence lengths: entry = seq | unit << 16, `q` units per workgroup.
// n == 0: every workgroup finds its start by a scan of the device arrays.
constexpr int kEvenTableMax = 1024;
struct EvenTable {
  int32_t n, q;
  uint32_t start[kEvenTableMax];
};

// Query tiles of a prefill launch listed by the host, heaviest (most keys to walk) first:
// entry = seq | tile << 16.  The hardware hands workgroups to free slots in id order, so a
// list sorted by work is longest-processing-time-first scheduling; a workgroup has its item
// after one scalar load.  n == 0: the kernel finds its item by a scan of the device arrays.
constexpr int kPfTableMax = 2048;
struct PfTable {
  int32_t n;
  uint32_t e[kPfTableMax];
};

// What the QKV projection needs to finish as rope_kv_write_kernel would (see oproj_kernels.hip).
struct RopeArgs {
  const int32_t *positions;
  const float *cos_sin;
  uint16_t *q_out;
  uint8_t *k_cache, *v_cache;
  const int64_t *slot_mapping;
  const float *k_scale, *v_scale;
  int64_t num_slots;
  int max_pos, Hq, Hkv, fp8;
};

// First key visible to any query row of a sequence, rounded down to a page boundary.
__host__ __device__ inline int kv_begin(int seq_len, int q_len, int window) {
  int p0 = seq_len - q_len;
  if (p0 < 0) p0 = 0;
  int lo = window > 0 ? p0 - window + 1 : 0;
  if (lo < 0) lo = 0;
  return lo & ~(kBlock - 1);
}

}  // namespace eid
