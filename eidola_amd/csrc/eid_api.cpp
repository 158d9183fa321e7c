// C ABI of the paged sink-attention library: argument validation (no HIP calls), launch
// planning (partition size, workspace layout) and dispatch to the gfx950 kernels.
#include <hip/hip_runtime.h>

#include "../../include/eidola_attn.h"
#ifdef EID_MEASURE
#include "../../include/eidola_attn_measure.h"
#endif
#include "eid_params.h"
#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

namespace eid {
hipError_t launch_splitkv(AttnParams &p, int ntiles, bool fp8, int32_t *plan_slot, hipStream_t st,
                          const ItemTable *tab = nullptr);
int splitkv_fill(int ntiles, bool fp8, int Hkv, bool pair = false, bool dma = false);
hipError_t launch_shortspan(const AttnParams &p, int ntiles, bool fp8, hipStream_t st,
                            const ItemTable *tab = nullptr);
hipError_t launch_even(AttnParams &p, int ntiles, bool fp8, int32_t *plan_slot, hipStream_t st,
                       const EvenTable *tab);
int even_wgs(int ntiles, bool fp8, int Hkv, bool pair, bool dma, bool all_cus);
bool shortspan_applies(int ntiles, bool fp8, long long num_items, int Hkv);
long long shortspan_items(int num_seqs, int nparts_max, long long sum_kv_len, int window);
hipError_t launch_prefill(const AttnParams &p, int num_q_tokens, bool fp8, hipStream_t st,
                          const PfTable *tab);
#ifdef EID_MEASURE
void set_timeline(void *buf, long long entries);
void set_kernel_events(void *start, void *stop);
void set_store_every_partition(int mode);
int store_every_partition_override();
#endif
bool build_prefill_table(const AttnParams &p, const int32_t *seq_lens_host,
                         const int32_t *cu_seqlens_q_host, PfTable *tab);
hipError_t launch_merge(const AttnParams &p, hipStream_t st);
hipError_t launch_rope_kv_write(const uint16_t *qkv, const int32_t *positions,
                                const float *cos_sin, int max_pos, uint16_t *q_out,
                                uint8_t *k_cache, uint8_t *v_cache, const int64_t *slot_mapping,
                                const float *k_scale, const float *v_scale, int Hq, int Hkv,
                                int64_t num_slots, int num_tokens, bool fp8, hipStream_t st);
int device_cus();
hipError_t static_scratch(uint8_t **ptr);
long long prefill_tiles_bound(int num_q_tokens, int num_seqs);
hipError_t launch_qkv_rope(const uint16_t *a, const uint16_t *w, const uint16_t *bias, int T, int K,
                           const RopeArgs &r, hipStream_t st);
hipError_t launch_o_proj(const uint16_t *a, const uint16_t *w, const uint16_t *bias,
                         const uint16_t *resid, uint16_t *out, int T, int N, int K,
                         hipStream_t st);
hipError_t launch_kv_write(const uint16_t *k_new, const uint16_t *v_new, uint8_t *k_cache,
                           uint8_t *v_cache, const int64_t *slot_mapping, const float *k_scale,
                           const float *v_scale, int Hkv, int64_t num_slots, int num_tokens,
                           bool fp8, hipStream_t st);
}  // namespace eid

static_assert(EID_STATIC_WORKSPACE_BYTES == eid::kStaticScratchBytes,
              "the header states the size of the static workspace");

namespace {
thread_local char g_err[512] = "";
}  // namespace

namespace eid {
// Records the thread-local error text of the library (shared with the scheduler's file).
int32_t set_error(int32_t status, const char *fmt, va_list ap) {
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  return status;
}
void clear_error() { g_err[0] = 0; }
}  // namespace eid

namespace {

int32_t fail(eid_status st, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  const int32_t rc = eid::set_error((int32_t)st, fmt, ap);
  va_end(ap);
  return rc;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Geometry checks shared by every entry point.
int32_t check_geometry(const eid_attn_desc *d) {
  if (!d) return fail(EID_ERR_INVALID_ARG, "desc is NULL");
  if (d->struct_size != sizeof(eid_attn_desc))
    return fail(EID_ERR_INVALID_ARG, "desc.struct_size %u != %zu", d->struct_size,
                sizeof(eid_attn_desc));
  if (d->head_dim != eid::kHeadDim)
    return fail(EID_ERR_UNSUPPORTED, "head_dim %d unsupported (64 only)", d->head_dim);
  if (d->block_size != eid::kBlock)
    return fail(EID_ERR_UNSUPPORTED, "block_size %d unsupported (16 only)", d->block_size);
  if (d->num_kv_heads <= 0 || d->num_q_heads <= 0)
    return fail(EID_ERR_INVALID_ARG, "head counts must be positive");
  if (d->num_q_heads != eid::kGroup * d->num_kv_heads)
    return fail(EID_ERR_UNSUPPORTED, "num_q_heads %d must be 8 * num_kv_heads %d",
                d->num_q_heads, d->num_kv_heads);
  const int h = d->num_kv_heads;
  if (!(h == 1 || h == 2 || h == 4 || h % 8 == 0))
    return fail(EID_ERR_UNSUPPORTED, "num_kv_heads %d must be 1, 2, 4 or a multiple of 8", h);
  if (d->kv_dtype != EID_KV_BF16 && d->kv_dtype != EID_KV_FP8_E4M3)
    return fail(EID_ERR_INVALID_ARG, "kv_dtype %d unknown", d->kv_dtype);
  if (d->num_blocks <= 0) return fail(EID_ERR_INVALID_ARG, "num_blocks must be positive");
  return EID_OK;
}

int32_t check_attn_desc(const eid_attn_desc *d) {
  int32_t rc = check_geometry(d);
  if (rc) return rc;
  if (d->num_seqs <= 0 || d->num_q_tokens <= 0)
    return fail(EID_ERR_INVALID_ARG, "num_seqs and num_q_tokens must be positive");
  if (d->num_seqs > 65535) return fail(EID_ERR_UNSUPPORTED, "num_seqs > 65535");
  if (d->max_q_len <= 0 || d->max_q_len > d->num_q_tokens)
    return fail(EID_ERR_INVALID_ARG, "max_q_len %d out of range", d->max_q_len);
  if (d->num_q_tokens < d->num_seqs)
    return fail(EID_ERR_INVALID_ARG, "num_q_tokens %d < num_seqs %d", d->num_q_tokens,
                d->num_seqs);
  if (d->max_kv_len <= 0) return fail(EID_ERR_INVALID_ARG, "max_kv_len must be positive");
  if (d->sum_kv_len != 0 && d->sum_kv_len < d->max_kv_len)
    return fail(EID_ERR_INVALID_ARG, "sum_kv_len %lld is below max_kv_len %d (0 = not known)",
                (long long)d->sum_kv_len, d->max_kv_len);
  if ((int64_t)d->max_blocks_per_seq * d->block_size < d->max_kv_len)
    return fail(EID_ERR_INVALID_ARG, "max_blocks_per_seq %d cannot hold max_kv_len %d",
                d->max_blocks_per_seq, d->max_kv_len);
  if (!(d->softmax_scale > 0.f) || !std::isfinite(d->softmax_scale))
    return fail(EID_ERR_INVALID_ARG, "softmax_scale must be finite and positive");
  if (d->window < 0) return fail(EID_ERR_INVALID_ARG, "window must be >= 0");
  if (d->partition_size != 0 &&
      (d->partition_size < 64 || d->partition_size > 4096 || d->partition_size % 64 != 0))
    return fail(EID_ERR_INVALID_ARG, "partition_size %d must be 0 or a multiple of 64 in [64,4096]",
                d->partition_size);
  return EID_OK;
}

struct Plan {
  int32_t partition, nparts_max, ws_rows;
  bool dynamic;
  size_t parts_bytes;            // per-sequence piece counts of an even split (run-time partition)
  size_t ml_bytes, acc_bytes;
  int32_t pf_splits;             // key-range parts per prefill tile (1 = no split)
  size_t pf_ml_bytes, pf_acc_bytes;
};

// Longest query a split-KV (verify) sequence may have in this call: 6 rows x 8 heads = three
// 16-row tiles; 8 rows = four tiles, or 16 rows = two waves of four tiles per KV head, when
// no sequence of the batch is longer than that (the prefill kernel's 32-token tile would be
// mostly empty for such sequences, and the batch is bandwidth-bound).
int32_t short_q_max(const eid_attn_desc *d) {
  // 9..16 rows: two waves per KV head, 8 rows each, both loading the head's K/V.  That doubles
  // the traffic through the CU's cache, so it pays only while the prefill kernel's workgroups
  // (one per sequence and KV head at these lengths) would not fill the device: 8 x 16 rows
  // behind 32k tokens 310 -> 182 us, 32 x 16 behind 8k 322 -> 194 us, 48 x 16 387 -> 300 us,
  // but 64 x 16 414 -> 427 us (left to the prefill kernel).  With four waves per KV head
  // (17..32 rows) the balance tips earlier: 2 x 20 rows behind 60k 296 -> 141 us, 8 x 24
  // behind 32k 330 -> 273 us, 8 x 32 358 -> 338 us, but 32 x 32 behind 8k 351 -> 360 us.
  if (d->max_q_len > eid::kShortQMaxRows && d->max_q_len <= eid::kShortQMaxRows4 &&
      d->num_kv_heads % 8 == 0 &&
      (long long)d->num_seqs * d->num_kv_heads <= eid::kRows4MaxGroups)
    return eid::kShortQMaxRows4;  // four waves per KV head: a handful of sequences only (below)
  if (d->max_q_len > eid::kShortQMaxWide && d->max_q_len <= eid::kShortQMaxRows &&
      d->num_kv_heads % 8 == 0 && (long long)d->num_seqs * d->num_kv_heads <= eid::kRowsMaxGroups)
    return eid::kShortQMaxRows;
  return d->max_q_len > eid::kShortQMax && d->max_q_len <= eid::kShortQMaxWide ? eid::kShortQMaxWide
                                                                                : eid::kShortQMax;
}
// 16-row tiles per KV head of the verify class: 3, 4, or 8 (two waves of four)
int verify_tiles(const eid_attn_desc *d) {
  const int32_t q = short_q_max(d);
  return q == eid::kShortQMaxRows4 ? 16 : q == eid::kShortQMaxRows ? 8 : q == eid::kShortQMaxWide ? 4 : 3;
}

// Longest key span a split-KV sequence can have (from its first visible page to its end).
int32_t max_span(const eid_attn_desc *d) {
  if (d->window > 0) {
    const int64_t w = (int64_t)d->window + short_q_max(d) + eid::kBlock - 1;
    return (int32_t)(w < d->max_kv_len ? w : d->max_kv_len);
  }
  return d->max_kv_len;
}

Plan make_plan(const eid_attn_desc *d) {
  Plan pl;
  const int32_t span = max_span(d);
  // partition_size == 0: the kernels size the partition from the batch at run time, never
  // below kDynPartitionMin, which therefore bounds the partition count for the workspace.
  int32_t P = d->partition_size ? d->partition_size : eid::kDynPartitionMin;
  pl.dynamic = d->partition_size == 0;
  // ... unless the host can already tell what they would choose: with at least one sequence
  // per CU and no span beyond the partition cap, every sequence is one work item.  Planning
  // it here makes the kernels map workgroup w to sequence w with no scan of seq_lens at all
  // (with hundreds of sequences the scans are a fifth of the run time) and no partials.
  if (pl.dynamic && d->num_seqs >= eid::device_cus() && span <= eid::kDynPartitionCap) {
    P = (span + 63) / 64 * 64;
    pl.dynamic = false;
  }
  // Small batches: when every 64-key chunk of the batch can have a wave of its own at once
  // (512-key partitions, one workgroup of eight waves per partition and KV head, all
  // resident together), the call is a few memory latencies long instead of a serial walk.
  if (pl.dynamic) {
    const long long items = eid::shortspan_items(
        d->num_seqs, (span + eid::kShortSpanMax - 1) / eid::kShortSpanMax, d->sum_kv_len, d->window);
    if (eid::shortspan_applies(d->max_q_len <= 2 ? 1 : verify_tiles(d), d->kv_dtype == EID_KV_FP8_E4M3, items,
                               d->num_kv_heads)) {
      P = eid::kShortSpanMax;
      pl.dynamic = false;
    }
  }
  pl.partition = P;
  pl.nparts_max = (span + P - 1) / P;
  // An even split cuts the launch into equal ranges of units, and the count of every sequence's
  // pieces goes through the workspace to the merge.  Run-time partition: the units are chunks
  // (ranges of at least P keys), and a range's ends fall anywhere in a sequence: one more
  // piece than whole partitions.
  pl.parts_bytes = 0;
  if (pl.nparts_max > 1) {
    if (pl.dynamic) pl.nparts_max += 1;
    pl.parts_bytes = ((size_t)d->num_seqs * sizeof(int32_t) + 255) / 256 * 256;
  }
  pl.ws_rows = std::min(d->max_q_len, short_q_max(d));
  const size_t cells = (size_t)d->num_seqs * pl.ws_rows * d->num_q_heads * pl.nparts_max;
  pl.ml_bytes = (cells * 2 * sizeof(float) + 255) / 256 * 256;
  pl.acc_bytes = (cells * eid::kHeadDim * sizeof(_Float16) + 255) / 256 * 256;
  // Prefill rows: when the query tiles alone cannot fill the device (two workgroups per CU)
  // and the context is long enough to share out, every tile's key range is split into parts
  // of at least 512 keys that run side by side and are merged afterwards.
  pl.pf_splits = 1;
  pl.pf_ml_bytes = pl.pf_acc_bytes = 0;
  if (d->max_q_len > short_q_max(d)) {
    const long long wgs = eid::prefill_tiles_bound(d->num_q_tokens, d->num_seqs) * d->num_kv_heads;
    // (aim: the split that comes nearest to one fill; two fills were measured too: better for
    // one 512-token chunk behind 60k tokens, worse for a 2,048-token chunk without a prior)
    const long long fill = 2LL * eid::device_cus(), w1 = wgs > 0 ? wgs : 1;
    const long long by_fill = (fill + w1 / 2) / w1, by_len = d->max_kv_len / 512;
    const long long ks = by_fill < by_len ? by_fill : by_len;
    pl.pf_splits = (int32_t)(ks < 1 ? 1 : ks > 8 ? 8 : ks);
    if (pl.pf_splits > 1) {
      const size_t pcells = (size_t)d->num_q_tokens * pl.pf_splits * d->num_q_heads;
      pl.pf_ml_bytes = (pcells * 2 * sizeof(float) + 255) / 256 * 256;
      pl.pf_acc_bytes = pcells * eid::kHeadDim * sizeof(_Float16);
    }
  }
  return pl;
}

int32_t check_attn_args(const eid_attn_desc *d, const eid_attn_args *a, bool need_q,
                        bool need_cu, bool need_ws = true) {
  if (!a) return fail(EID_ERR_INVALID_ARG, "args is NULL");
  if (need_q && (!a->q || !a->k_cache || !a->v_cache || !a->block_table))
    return fail(EID_ERR_INVALID_ARG, "q, k_cache, v_cache and block_table must be non-NULL");
  if (!a->out || !a->seq_lens) return fail(EID_ERR_INVALID_ARG, "out and seq_lens must be non-NULL");
  if (need_cu && !a->cu_seqlens_q) return fail(EID_ERR_INVALID_ARG, "cu_seqlens_q is NULL");
  if (!aligned16(a->q) || !aligned16(a->out) || !aligned16(a->k_cache) || !aligned16(a->v_cache))
    return fail(EID_ERR_INVALID_ARG, "q, out, k_cache and v_cache must be 16-byte aligned");
  if (d->kv_dtype == EID_KV_FP8_E4M3 && need_q && (!a->k_scale || !a->v_scale))
    return fail(EID_ERR_INVALID_ARG, "fp8 KV needs k_scale and v_scale");
  if (!need_ws) return EID_OK;
  const Plan pl = make_plan(d);
  const size_t need =
      eid::kPlanBytes + pl.parts_bytes + pl.ml_bytes + pl.acc_bytes + pl.pf_ml_bytes + pl.pf_acc_bytes;
  if (!a->workspace || a->workspace_bytes < need)
    return fail(EID_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need,
                a->workspace ? a->workspace_bytes : (size_t)0);
  if ((reinterpret_cast<uintptr_t>(a->workspace) & 255u) != 0)
    return fail(EID_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  return EID_OK;
}

eid::AttnParams make_params(const eid_attn_desc *d, const eid_attn_args *a, const Plan &pl) {
  eid::AttnParams p;
  std::memset(&p, 0, sizeof p);
  p.q = static_cast<const uint16_t *>(a->q);
  p.out = static_cast<uint16_t *>(a->out);
  p.lse = a->lse;
  p.k_cache = static_cast<const uint8_t *>(a->k_cache);
  p.v_cache = static_cast<const uint8_t *>(a->v_cache);
  p.block_table = a->block_table;
  p.cu_seqlens_q = a->cu_seqlens_q;
  p.seq_lens = a->seq_lens;
  p.sinks = a->sinks;
  p.k_scale = a->k_scale;
  p.v_scale = a->v_scale;
  p.k_new = nullptr;  // set by eid_attn_decode only
  p.v_new = nullptr;
  uint8_t *ws = static_cast<uint8_t *>(a->workspace);
  p.plan = nullptr;
  p.plan_slot = nullptr;
  const size_t head = eid::kPlanBytes + pl.parts_bytes;  // plan slots, then the piece counts
  p.seq_parts = reinterpret_cast<int32_t *>(ws + eid::kPlanBytes);
  p.ws_ml = reinterpret_cast<float *>(ws + head);
  p.ws_acc = reinterpret_cast<_Float16 *>(ws + head + pl.ml_bytes);
  p.pf_splits = pl.pf_splits;
  p.pf_ml = reinterpret_cast<float *>(ws + head + pl.ml_bytes + pl.acc_bytes);
  p.pf_acc = reinterpret_cast<_Float16 *>(ws + head + pl.ml_bytes + pl.acc_bytes + pl.pf_ml_bytes);
  p.num_q_tokens = d->num_q_tokens;
  p.sum_kv_len = d->sum_kv_len;
  p.num_seqs = d->num_seqs;
  p.num_q_heads = d->num_q_heads;
  p.num_kv_heads = d->num_kv_heads;
  p.max_blocks_per_seq = d->max_blocks_per_seq;
  p.last_block = (int32_t)std::min<int64_t>(d->num_blocks - 1, 0x7fffffff);
  p.window = d->window;
  p.partition = pl.partition;
  p.dynamic_partition = pl.dynamic ? 1 : 0;
  p.target_items = 512;
  p.nparts_max = pl.nparts_max;
  p.ws_rows = pl.ws_rows;
  p.softmax_scale = d->softmax_scale;
  return p;
}

// Helper stream of the calling thread on the current device: the prefill launch of a mixed
// batch runs there, beside the split-KV launches on the caller's stream (fork and join by
// events, so the caller sees one stream's worth of ordering).  Created on first use at the
// default priority and kept for the life of the thread; nullptr if creation fails (the call
// then runs its launches one after the other).
struct Helper {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  bool tried = false, ok = false;
  ~Helper() {  // the owning thread ends: give the stream and the events back
    if (fork) (void)hipEventDestroy(fork);
    if (join) (void)hipEventDestroy(join);
    if (stream) (void)hipStreamDestroy(stream);
  }
};

// Joins the helper stream back into the caller's stream when it goes out of scope, on error
// returns as on success, so that no launch stays behind on the helper stream that the caller's
// stream never waits for (under capture: no unjoined fork).
struct HelperJoin {
  Helper *hs = nullptr;
  hipStream_t st = nullptr;
  bool forked = false;
  hipError_t join() {
    if (!forked) return hipSuccess;
    forked = false;
    hipError_t e = hipEventRecord(hs->join, hs->stream);
    if (e == hipSuccess) e = hipStreamWaitEvent(st, hs->join, 0);
    return e;
  }
  ~HelperJoin() { (void)join(); }
};
Helper *helper_stream() {
  constexpr int kMaxDevices = 64;
  thread_local Helper helpers[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  Helper &h = helpers[dev];
  if (!h.tried) {
    h.tried = true;
    h.ok = hipStreamCreateWithFlags(&h.stream, hipStreamNonBlocking) == hipSuccess &&
           hipEventCreateWithFlags(&h.fork, hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&h.join, hipEventDisableTiming) == hipSuccess;
    if (!h.ok) (void)hipGetLastError();  // not sticky: the sequential path follows
  }
  return h.ok ? &h : nullptr;
}

// Whether the short-span kernel serves the split-KV rows of a call (q_len class of `ntiles`
// 16-row tiles): spans within one workgroup's reach, or partitions of exactly that size, and
// few enough of them.
bool use_shortspan(const eid_attn_desc *d, const Plan &pl, int ntiles) {
  if (pl.nparts_max == 1 ? max_span(d) > eid::kShortSpanMax
                         : (pl.dynamic || pl.partition != eid::kShortSpanMax))
    return false;
  return eid::shortspan_applies(
      ntiles, d->kv_dtype == EID_KV_FP8_E4M3,
      eid::shortspan_items(d->num_seqs, pl.nparts_max, d->sum_kv_len, d->window), d->num_kv_heads);
}

int32_t hip_fail(hipError_t e, const char *what) {
  return fail(EID_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

// Whether work enqueued on `st` right now is being recorded into a HIP graph.  A plan made
// from the caller's HOST copies of the lengths (exact grids, the partition size, the item
// list passed by value) would be frozen into the graph and silently go stale when the device
// arrays change between replays, so under capture the host copies are ignored and the
// kernels plan from the device arrays, as they do without them.
// A failed query (the legacy stream while another stream captures in global mode, say) counts
// as capturing: the launch is then sized from the descriptor, which is right in either case,
// where a plan from the host copies frozen into somebody's graph would not be.
bool stream_is_capturing(hipStream_t st) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &status) != hipSuccess) {
    (void)hipGetLastError();
    return true;
  }
  return status != hipStreamCaptureStatusNone;
}

// ---- opt-in checks of what the library otherwise has to take on trust (EID_DEBUG=1) -----
// The host copies of the length arrays and of the block table must equal the device arrays,
// and desc.sum_kv_len must not be below the true sum: a mismatch makes the kernels drop or
// misplace work without any error.  With EID_DEBUG set in the environment the attention entry
// points copy the device arrays back (after waiting for the stream) and compare.  Slow, and
// not possible on a capturing stream; meant for bring-up of an engine's scheduler.
bool debug_checks_on() {
  static const bool on = getenv("EID_DEBUG") != nullptr;
  return on;
}

int32_t debug_check_host_copies(const eid_attn_desc *d, const eid_attn_args *a, bool decode,
                                hipStream_t st) {
  hipError_t e = hipStreamSynchronize(st);
  if (e != hipSuccess) return hip_fail(e, "EID_DEBUG: stream synchronize");
  try {
    const size_t S = (size_t)d->num_seqs;
    std::vector<int32_t> lens(S);
    e = hipMemcpy(lens.data(), a->seq_lens, S * sizeof(int32_t), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "EID_DEBUG: copy of seq_lens");
    long long sum = 0;
    for (size_t s = 0; s < S; ++s) {
      sum += lens[s];
      if (lens[s] > d->max_kv_len)
        return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: seq_lens[%zu] = %d exceeds desc.max_kv_len %d", s,
                    lens[s], d->max_kv_len);
      if (a->seq_lens_host && a->seq_lens_host[s] != lens[s])
        return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: seq_lens_host[%zu] = %d, device holds %d", s,
                    a->seq_lens_host[s], lens[s]);
    }
    if (d->sum_kv_len != 0 && d->sum_kv_len < sum)
      return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: desc.sum_kv_len %lld is below the sum of seq_lens %lld",
                  (long long)d->sum_kv_len, sum);
    if (!decode && a->cu_seqlens_q_host) {
      std::vector<int32_t> cu(S + 1);
      e = hipMemcpy(cu.data(), a->cu_seqlens_q, (S + 1) * sizeof(int32_t), hipMemcpyDeviceToHost);
      if (e != hipSuccess) return hip_fail(e, "EID_DEBUG: copy of cu_seqlens_q");
      for (size_t s = 0; s <= S; ++s)
        if (a->cu_seqlens_q_host[s] != cu[s])
          return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: cu_seqlens_q_host[%zu] = %d, device holds %d", s,
                      a->cu_seqlens_q_host[s], cu[s]);
    }
    if (decode && a->block_table_host) {
      const size_t mb = (size_t)d->max_blocks_per_seq;
      std::vector<int32_t> bt(S * mb);
      e = hipMemcpy(bt.data(), a->block_table, S * mb * sizeof(int32_t), hipMemcpyDeviceToHost);
      if (e != hipSuccess) return hip_fail(e, "EID_DEBUG: copy of block_table");
      for (size_t s = 0; s < S; ++s) {
        const size_t used = ((size_t)std::max(lens[s], 0) + eid::kBlock - 1) / eid::kBlock;
        for (size_t j = 0; j < used && j < mb; ++j)
          if (a->block_table_host[s * mb + j] != bt[s * mb + j])
            return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: block_table_host[%zu][%zu] = %d, device holds %d",
                        s, j, a->block_table_host[s * mb + j], bt[s * mb + j]);
      }
    }
  } catch (...) {
    return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: out of host memory");
  }
  return EID_OK;
}

// ---- launch planning from the caller's host copies of seq_lens / cu_seqlens_q ----------

// Key spans of the sequences of one q_len class, as the kernels see them (view_seq).  The
// three arrays live in storage the caller provides (num_seqs entries each).
struct ClassSpans {
  int32_t *spans = nullptr, *seq = nullptr, *len = nullptr;  // span, index, length per sequence
  size_t n = 0;
  long long total = 0;
  int32_t longest = 0;
  long long items(int32_t P, int32_t nparts_max) const {
    long long c = 0;
    for (size_t i = 0; i < n; ++i) c += std::min((spans[i] + P - 1) / P, nparts_max);
    return c;
  }
};

ClassSpans class_spans(const eid_attn_desc *d, const int32_t *seq_lens, const int32_t *cu,
                       int32_t ws_rows, int32_t qlen_lo, int32_t qlen_hi, int32_t *storage) {
  ClassSpans c;
  c.spans = storage;
  c.seq = storage + d->num_seqs;
  c.len = storage + 2 * (size_t)d->num_seqs;
  for (int32_t s = 0; s < d->num_seqs; ++s) {
    const int32_t L = std::min<int64_t>(seq_lens[s], (int64_t)d->max_blocks_per_seq * eid::kBlock);
    const int32_t qlen = cu ? cu[s + 1] - cu[s] : 1;
    if (qlen < qlen_lo || qlen > qlen_hi || qlen > ws_rows || L < qlen) continue;
    const int32_t span = L - eid::kv_begin(L, qlen, d->window);
    if (span <= 0) continue;
    c.spans[c.n] = span;
    c.seq[c.n] = s;
    c.len[c.n] = L;
    ++c.n;
    c.total += span;
    c.longest = std::max(c.longest, span);
  }
  return c;
}

// The partition the kernels' run-time rule would derive for these spans (the same tiers in the
// same order: one workgroup per CU, one device fill, whole sequences, equal pieces of nearly
// uniform batches, about three fills), computed once here instead of by every workgroup.
int32_t host_partition(const ClassSpans &c, long long T, long long Tlo, int32_t Pmin,
                       int32_t nparts_max) {
  const long long active = (long long)c.n, cap = eid::kDynPartitionCap;
  auto up64 = [](long long v) { return (v + 63) / 64 * 64; };
  auto single_fill = [&](const long long Tx) -> int32_t {
    if (active > Tx) return 0;
    long long hi = up64(c.longest);
    if (active < Tx) hi = std::min(hi, up64((c.total + (Tx - active) - 1) / (Tx - active)));
    hi = std::max(hi, (long long)Pmin);
    if (hi >= cap) return 0;
    int32_t lo_i = Pmin / 64, hi_i = (int32_t)hi / 64 - 1, P = (int32_t)hi;
    while (lo_i <= hi_i) {
      const int32_t mid = (lo_i + hi_i) >> 1;
      if (c.items(mid * 64, nparts_max) <= Tx) {
        P = mid * 64;
        hi_i = mid - 1;
      } else {
        lo_i = mid + 1;
      }
    }
    return P;
  };
  if (Tlo < T)
    if (const int32_t P = single_fill(std::max(Tlo, 1LL))) return P;
  if (const int32_t P = single_fill(T)) return P;
  const long long whole = up64(c.longest);
  if (active >= Tlo && whole <= cap) return (int32_t)std::max(whole, (long long)Pmin);
  if ((long long)c.longest * active * 4 <= c.total * 5) {
    const long long pieces = (c.longest + cap - 1) / cap;
    return (int32_t)std::max(up64((c.longest + pieces - 1) / pieces), (long long)Pmin);
  }
  return (int32_t)std::min(cap, std::max((long long)eid::kDynPartitionFloor, up64(c.total / (3 * T))));
}

// What the host decided for the split-KV launch of one q_len class.
struct ClassPlan {
  bool skip = false;      // no sequence of this class: launch nothing
  bool short_span = false;
  bool merge = false;     // some sequence has more than one partition
  bool even = false;      // even split: equal contiguous ranges of the launch's units
};

// EID_EVEN=0 switches the even split off (the launches then take one workgroup per item), for
// A/B measurements.
bool even_allowed() {
  static const bool on = [] {
    const char *e = getenv("EID_EVEN");
    return !(e && atoi(e) == 0);
  }();
  return on;
}

// Sets p.partition / p.dynamic_partition / p.exact_items for the class [qlen_lo, qlen_hi] and
// says which kernel serves it.  Without host lengths this is the plan made from the
// descriptor alone; with them, the run-time choices of the kernels are made here.
// `no_heap`: the call must not allocate (host memory included): batches beyond the stack
// storage are then left to the kernels' own planning.
ClassPlan plan_class(const eid_attn_desc *d, const eid_attn_args *a, const Plan &pl,
                     eid::AttnParams &p, int ntiles, int32_t qlen_lo, int32_t qlen_hi,
                     bool decode, eid::EvenTable *etab, eid::ItemTable *table = nullptr,
                     bool no_heap = false, bool capturing = false) {
  ClassPlan cp;
  if (table) table->n = table->has_blk = 0;
  etab->n = etab->q = 0;
  const bool fp8 = d->kv_dtype == EID_KV_FP8_E4M3;
  p.qlen_lo = qlen_lo;
  p.qlen_hi = qlen_hi;
  p.partition = pl.partition;
  p.dynamic_partition = pl.dynamic ? 1 : 0;
  p.exact_items = 0;
  // bf16 cache and no prefill launch beside this one: the chunks stream in by direct global -> LDS loads
  static const bool no_dma = getenv("EID_NO_DMA") != nullptr;  // for A/B measurements
  p.dma = (!fp8 && !p.share_cus && !no_dma) ? 1 : 0;
  p.dma_pair = (fp8 && p.fp8_pair && ntiles == 1 && !p.share_cus && !no_dma) ? 1 : 0;
  p.dma_fp8 = (fp8 && ntiles >= 3 && !p.share_cus && !no_dma) ? 1 : 0;
  p.target_items = eid::splitkv_fill(ntiles, fp8, d->num_kv_heads, p.fp8_pair != 0, p.dma != 0);
  cp.short_span = use_shortspan(d, pl, ntiles);
  cp.merge = pl.nparts_max > 1;
  constexpr int32_t kHostPlanMaxSeqs = 8192;  // beyond that the host pass is no longer free
  const int32_t *cu = decode ? nullptr : a->cu_seqlens_q_host;
  // even split: one row group per KV head (no sequence of the class has more rows than a wave takes)
  const bool even_ok = even_allowed() && pl.nparts_max > 1 && !cp.short_span &&
                       (ntiles == 1 || ntiles == 3 || ntiles == 4);
  static const bool every = getenv("EID_STORE_EVERY_PARTITION") != nullptr;  // measurement aid
  p.store_every_partition = every ? 1 : 0;
#ifdef EID_MEASURE
  if (eid::store_every_partition_override() >= 0) p.store_every_partition = eid::store_every_partition_override();
#endif
  p.even_wgs = even_ok ? eid::even_wgs(ntiles, fp8, d->num_kv_heads, p.fp8_pair != 0, p.dma != 0 || p.dma_pair != 0,
                                       p.store_every_partition != 0 && !pl.dynamic)
                       : 0;
  if (p.mixed_wgs > 0 && p.even_wgs > p.mixed_wgs) p.even_wgs = p.mixed_wgs;
  if (!a->seq_lens_host || (!decode && !cu) || d->num_seqs > kHostPlanMaxSeqs || capturing) {
    // Without the lengths: a run-time partition always takes the even split (every workgroup
    // finds its range by a scan of the device arrays); the caller's partition takes it when
    // the bound on its items says that the launch is several device fills long.
    if (even_ok) {
      const long long span_sum = d->sum_kv_len > 0 && d->window == 0
                                     ? d->sum_kv_len : (long long)d->num_seqs * max_span(d);
      cp.even = pl.dynamic || span_sum / pl.partition + d->num_seqs >= 4LL * p.even_wgs;
    }
    return cp;
  }
  int32_t stack_store[3 * eid::kStackPlanSeqs];  // 12 KiB: most batches need no heap at all
  std::vector<int32_t> heap_store;
  int32_t *store = stack_store;
  if (d->num_seqs > eid::kStackPlanSeqs) {
    if (no_heap) return cp;
    try {
      heap_store.resize(3 * (size_t)d->num_seqs);
    } catch (...) {  // out of host memory: nothing may cross the C ABI; the kernels plan instead
      return cp;
    }
    store = heap_store.data();
  }
  const ClassSpans c = class_spans(d, a->seq_lens_host, cu, pl.ws_rows, qlen_lo, qlen_hi, store);
  if (c.n == 0) {
    cp.skip = true;
    return cp;
  }
  if (pl.nparts_max == 1) return cp;  // workgroup w serves sequence w: nothing to refine
  const bool small_batch = pl.dynamic && eid::shortspan_applies(ntiles, fp8, c.items(eid::kShortSpanMax, pl.nparts_max),
                                                                d->num_kv_heads);
  // Even split: the launch's units (chunks, or partitions of the caller's size when there are
  // at least two of them per workgroup) cut into equal contiguous ranges, one per workgroup.
  const long long U = pl.dynamic ? eid::kChunk : pl.partition;
  if (even_ok && !small_batch) {
    long long C = 0;
    for (size_t i = 0; i < c.n; ++i)
      C += pl.dynamic ? (c.spans[i] + U - 1) / U : std::min<long long>((c.spans[i] + U - 1) / U, pl.nparts_max);
    const long long G = p.even_wgs;
    const long long q = std::max<long long>((C + G - 1) / G, pl.dynamic ? eid::kEvenMinChunks : 1);
    const long long n = (C + q - 1) / q;
    if (pl.dynamic || (C >= 2 * G && !(decode && table && C <= eid::kItemTableMax))) {
      cp.even = true;
      p.exact_items = n;
      // where every workgroup's range starts, and whether any sequence is cut
      bool cut = false;
      long long pos = 0;  // units before sequence i
      for (size_t i = 0; i < c.n; ++i) {
        const long long n_s = pl.dynamic ? (c.spans[i] + U - 1) / U
                                         : std::min<long long>((c.spans[i] + U - 1) / U, pl.nparts_max);
        if (p.store_every_partition && !pl.dynamic) cut = cut || n_s > 1;
        else cut = cut || pos / q != (pos + n_s - 1) / q;
        if (n <= eid::kEvenTableMax && c.seq[i] <= 0xffff)
          for (long long b = (pos + q - 1) / q; b * q < pos + n_s; ++b)
            etab->start[b] = (uint32_t)c.seq[i] | (uint32_t)(b * q - pos) << 16;
        pos += n_s;
      }
      if (n <= eid::kEvenTableMax && (long long)d->max_kv_len / U + 1 < 0xffff && d->num_seqs <= 0xffff) {
        etab->n = (int32_t)n;
        etab->q = (int32_t)q;
      }
      cp.merge = cut;
      return cp;
    }
  }
  if (pl.dynamic) {
    if (small_batch) {
      cp.short_span = true;  // small batch: one wave per chunk (see make_plan)
      p.partition = eid::kShortSpanMax;
    } else {
      const long long T = p.target_items;
      p.partition = host_partition(c, T, std::min<long long>(T, eid::device_cus()), pl.partition,
                                   pl.nparts_max);
    }
    p.dynamic_partition = 0;
  }
  p.exact_items = c.items(p.partition, pl.nparts_max);
  cp.merge = p.exact_items > (long long)c.n;
  // Few items of a decode launch: list them for the kernels (sequence-major, as they would
  // find them themselves)
  static const bool no_table = getenv("EID_NO_ITEM_TABLE") != nullptr;  // for A/B measurements
  if (table && decode && !no_table && p.exact_items <= eid::kItemTableMax) {
    int32_t n = 0;
    const int32_t *bth = a->block_table_host;
    for (size_t i = 0; i < c.n; ++i) {
      const int32_t parts = std::min((c.spans[i] + p.partition - 1) / p.partition, pl.nparts_max);
      const int32_t L = c.len[i], kb = eid::kv_begin(L, 1, d->window);
      for (int32_t part = 0; part < parts; ++part) {
        if (bth) {  // the ids the kernel would fetch for the item's first chunk (see attend)
          const int32_t t0 = kb + part * p.partition, t1 = std::min(t0 + p.partition, L);
          const int32_t last = (t1 + eid::kBlock - 1) / eid::kBlock - 1;
          for (int32_t b = 0; b < 4; ++b)
            table->blk[n][b] = bth[(size_t)c.seq[i] * d->max_blocks_per_seq +
                                   std::min(t0 / eid::kBlock + b, last)];
        }
        table->e[n++] = (unsigned long long)(uint32_t)c.seq[i] | (unsigned long long)part << 16 |
                        (unsigned long long)(uint32_t)L << 32;
      }
    }
    table->n = n;
    table->has_blk = bth ? 1 : 0;
  }
  return cp;
}

}  // namespace

extern "C" {

uint32_t eid_version(void) { return (EID_VERSION_MAJOR << 16) | EID_VERSION_MINOR; }

const char *eid_last_error(void) { return g_err; }

#ifdef EID_MEASURE
void eid_debug_set_timeline(void *device_buf, int64_t entries) { eid::set_timeline(device_buf, entries); }

void eid_debug_set_kernel_events(void *start_event, void *stop_event) {
  eid::set_kernel_events(start_event, stop_event);
}

void eid_debug_set_store_every_partition(int32_t mode) { eid::set_store_every_partition(mode); }
#endif

int32_t eid_partition_size(const eid_attn_desc *desc) {
  if (check_attn_desc(desc)) return 0;
  return make_plan(desc).partition;
}

size_t eid_workspace_bytes(const eid_attn_desc *desc) {
  if (check_attn_desc(desc)) return 0;
  const Plan pl = make_plan(desc);
  return eid::kPlanBytes + pl.parts_bytes + pl.ml_bytes + pl.acc_bytes + pl.pf_ml_bytes + pl.pf_acc_bytes;
}

int32_t eid_kv_write(const eid_attn_desc *desc, const void *k_new, const void *v_new,
                     void *k_cache, void *v_cache, const int64_t *slot_mapping,
                     int32_t num_tokens, const float *k_scale, const float *v_scale,
                     void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_geometry(desc)) return rc;
  if (num_tokens < 0) return fail(EID_ERR_INVALID_ARG, "num_tokens %d < 0", num_tokens);
  if (num_tokens == 0) return EID_OK;
  if (!k_new || !v_new || !k_cache || !v_cache || !slot_mapping)
    return fail(EID_ERR_INVALID_ARG, "k_new, v_new, k_cache, v_cache, slot_mapping must be non-NULL");
  if (!aligned16(k_new) || !aligned16(v_new) || !aligned16(k_cache) || !aligned16(v_cache))
    return fail(EID_ERR_INVALID_ARG, "k_new, v_new, k_cache and v_cache must be 16-byte aligned");
  const bool fp8 = desc->kv_dtype == EID_KV_FP8_E4M3;
  if (fp8 && (!k_scale || !v_scale)) return fail(EID_ERR_INVALID_ARG, "fp8 KV needs k_scale and v_scale");
  if (debug_checks_on() && !stream_is_capturing(static_cast<hipStream_t>(hip_stream))) {
    // duplicate slots in one call are undefined behaviour (two rows race for one cache row)
    hipError_t de = hipStreamSynchronize(static_cast<hipStream_t>(hip_stream));
    if (de != hipSuccess) return hip_fail(de, "EID_DEBUG: stream synchronize");
    try {
      std::vector<int64_t> slots((size_t)num_tokens);
      de = hipMemcpy(slots.data(), slot_mapping, slots.size() * sizeof(int64_t), hipMemcpyDeviceToHost);
      if (de != hipSuccess) return hip_fail(de, "EID_DEBUG: copy of slot_mapping");
      std::sort(slots.begin(), slots.end());
      for (size_t i = 1; i < slots.size(); ++i)
        if (slots[i] >= 0 && slots[i] == slots[i - 1])
          return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: slot %lld appears more than once in slot_mapping",
                      (long long)slots[i]);
    } catch (...) {
      return fail(EID_ERR_INVALID_ARG, "EID_DEBUG: out of host memory");
    }
  }
  hipError_t e = eid::launch_kv_write(
      static_cast<const uint16_t *>(k_new), static_cast<const uint16_t *>(v_new),
      static_cast<uint8_t *>(k_cache), static_cast<uint8_t *>(v_cache), slot_mapping, k_scale,
      v_scale, desc->num_kv_heads, desc->num_blocks * desc->block_size, num_tokens, fp8,
      static_cast<hipStream_t>(hip_stream));
  if (e != hipSuccess) return hip_fail(e, "kv_write launch");
  return EID_OK;
}

int32_t eid_rope_kv_write(const eid_attn_desc *desc, const void *qkv, const int32_t *positions,
                          const float *cos_sin, int32_t max_pos, void *q_out, void *k_cache,
                          void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                          const float *k_scale, const float *v_scale, void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_geometry(desc)) return rc;
  if (4 * (desc->num_q_heads + 2 * desc->num_kv_heads) > 1024)
    return fail(EID_ERR_UNSUPPORTED, "num_kv_heads %d too large for one workgroup per token",
                desc->num_kv_heads);
  if (num_tokens < 0) return fail(EID_ERR_INVALID_ARG, "num_tokens %d < 0", num_tokens);
  if (max_pos <= 0) return fail(EID_ERR_INVALID_ARG, "max_pos %d must be positive", max_pos);
  if (num_tokens == 0) return EID_OK;
  if (!qkv || !positions || !cos_sin || !q_out || !k_cache || !v_cache || !slot_mapping)
    return fail(EID_ERR_INVALID_ARG,
                "qkv, positions, cos_sin, q_out, k_cache, v_cache, slot_mapping must be non-NULL");
  if (!aligned16(qkv) || !aligned16(cos_sin) || !aligned16(q_out) || !aligned16(k_cache) ||
      !aligned16(v_cache))
    return fail(EID_ERR_INVALID_ARG, "qkv, cos_sin, q_out, k_cache and v_cache must be 16-byte aligned");
  const bool fp8 = desc->kv_dtype == EID_KV_FP8_E4M3;
  if (fp8 && (!k_scale || !v_scale)) return fail(EID_ERR_INVALID_ARG, "fp8 KV needs k_scale and v_scale");
  hipError_t e = eid::launch_rope_kv_write(
      static_cast<const uint16_t *>(qkv), positions, cos_sin, max_pos,
      static_cast<uint16_t *>(q_out), static_cast<uint8_t *>(k_cache),
      static_cast<uint8_t *>(v_cache), slot_mapping, k_scale, v_scale, desc->num_q_heads,
      desc->num_kv_heads, desc->num_blocks * desc->block_size, num_tokens, fp8,
      static_cast<hipStream_t>(hip_stream));
  if (e != hipSuccess) return hip_fail(e, "rope_kv_write launch");
  return EID_OK;
}

int32_t eid_qkv_rope_kv_write(const eid_attn_desc *desc, const void *hidden, const void *weight,
                              const void *bias, int32_t in_features, const int32_t *positions,
                              const float *cos_sin, int32_t max_pos, void *q_out, void *k_cache,
                              void *v_cache, const int64_t *slot_mapping, int32_t num_tokens,
                              const float *k_scale, const float *v_scale, void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_geometry(desc)) return rc;
  if (num_tokens < 0) return fail(EID_ERR_INVALID_ARG, "num_tokens %d < 0", num_tokens);
  if (num_tokens > 64)
    return fail(EID_ERR_UNSUPPORTED, "num_tokens %d > 64: use eid_o_proj, then eid_rope_kv_write",
                num_tokens);
  if (max_pos <= 0) return fail(EID_ERR_INVALID_ARG, "max_pos %d must be positive", max_pos);
  if (in_features <= 0 || in_features % 64 != 0)
    return fail(EID_ERR_INVALID_ARG, "in_features %d must be a positive multiple of 64", in_features);
  if (num_tokens == 0) return EID_OK;
  if (!hidden || !weight || !positions || !cos_sin || !q_out || !k_cache || !v_cache || !slot_mapping)
    return fail(EID_ERR_INVALID_ARG, "hidden, weight, positions, cos_sin, q_out, k_cache, v_cache, "
                                     "slot_mapping must be non-NULL");
  if (!aligned16(hidden) || !aligned16(weight) || !aligned16(cos_sin) || !aligned16(q_out) ||
      !aligned16(k_cache) || !aligned16(v_cache))
    return fail(EID_ERR_INVALID_ARG,
                "hidden, weight, cos_sin, q_out, k_cache and v_cache must be 16-byte aligned");
  const bool fp8 = desc->kv_dtype == EID_KV_FP8_E4M3;
  if (fp8 && (!k_scale || !v_scale)) return fail(EID_ERR_INVALID_ARG, "fp8 KV needs k_scale and v_scale");
  eid::RopeArgs r;
  r.positions = positions;
  r.cos_sin = cos_sin;
  r.q_out = static_cast<uint16_t *>(q_out);
  r.k_cache = static_cast<uint8_t *>(k_cache);
  r.v_cache = static_cast<uint8_t *>(v_cache);
  r.slot_mapping = slot_mapping;
  r.k_scale = k_scale;
  r.v_scale = v_scale;
  r.num_slots = desc->num_blocks * desc->block_size;
  r.max_pos = max_pos;
  r.Hq = desc->num_q_heads;
  r.Hkv = desc->num_kv_heads;
  r.fp8 = fp8 ? 1 : 0;
  hipError_t e = eid::launch_qkv_rope(static_cast<const uint16_t *>(hidden),
                                      static_cast<const uint16_t *>(weight),
                                      static_cast<const uint16_t *>(bias), num_tokens, in_features, r,
                                      static_cast<hipStream_t>(hip_stream));
  if (e != hipSuccess) return hip_fail(e, "qkv_rope_kv_write launch");
  return EID_OK;
}

// Decode rows over an fp8 cache: a wave of the split-KV kernel takes two neighbouring KV
// heads, so that its loads cover whole 128-byte lines of a token row (one head's 64 fp8
// bytes are half a line).  Needs one query row per sequence (the 16 rows of a wave's tile
// are then the 16 query heads of the pair) and KV heads in groups of eight.
static bool fp8_pair_applies(const eid_attn_desc *d) {
  static const bool off = getenv("EID_NO_FP8_PAIR") != nullptr;  // for A/B measurements
  return !off && d->kv_dtype == EID_KV_FP8_E4M3 && d->max_q_len == 1 && d->num_kv_heads % 8 == 0;
}

// Decode call on validated arguments whose workspace is in place (the caller's, or the
// library's own static array).
static int32_t decode_launch(const eid_attn_desc *desc, const eid_attn_args *args, void *hip_stream,
                             bool no_heap) {
  const Plan pl = make_plan(desc);
  eid::AttnParams p = make_params(desc, args, pl);
  p.cu_seqlens_q = nullptr;  // one row per sequence by contract
  if ((args->k_new != nullptr) != (args->v_new != nullptr))
    return fail(EID_ERR_INVALID_ARG, "k_new and v_new must both be given or both be NULL");
  if (!aligned16(args->k_new) || !aligned16(args->v_new))
    return fail(EID_ERR_INVALID_ARG, "k_new and v_new must be 16-byte aligned");
  p.k_new = static_cast<const uint16_t *>(args->k_new);  // fused write of the newest token
  p.v_new = static_cast<const uint16_t *>(args->v_new);
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const bool fp8 = desc->kv_dtype == EID_KV_FP8_E4M3;
  const bool capturing = stream_is_capturing(st);
  if (debug_checks_on() && !capturing && !no_heap)
    if (int32_t rc = debug_check_host_copies(desc, args, true, st)) return rc;
  p.fp8_pair = fp8_pair_applies(desc) ? 1 : 0;
  int32_t *plan_slots = static_cast<int32_t *>(args->workspace);
  eid::ItemTable table;  // (8 KiB on the stack; only `n` entries are ever read)
  eid::EvenTable etab;   // (4 KiB)
  const ClassPlan cp = plan_class(desc, args, pl, p, 1, 1, 1, true, &etab, &table, no_heap, capturing);
  if (cp.skip) return EID_OK;  // (every sequence empty or malformed: nothing is written)
  const eid::ItemTable *tab = table.n > 0 ? &table : nullptr;
  // spans of at most 8 chunks, or a small batch in partitions of that size: one workgroup
  // per (sequence, partition, KV head), a chunk per wave
  if (cp.short_span) p.plan_slot = plan_slots;  // (the kernel records its partition there)
  hipError_t e = cp.even         ? eid::launch_even(p, 1, fp8, plan_slots, st, &etab)
                 : cp.short_span ? eid::launch_shortspan(p, 1, fp8, st, tab)
                                 : eid::launch_splitkv(p, 1, fp8, plan_slots, st, tab);
  if (cp.short_span) p.plan_slot = nullptr;     // (the merge of this call takes p.partition)
  if (e != hipSuccess) return hip_fail(e, "split-KV launch");
  if (args->split_done_event) {
    e = hipEventRecord(static_cast<hipEvent_t>(args->split_done_event), st);
    if (e != hipSuccess) return hip_fail(e, "split_done_event record");
  }
  if (cp.merge) {
    e = eid::launch_merge(p, st);
    if (e != hipSuccess) return hip_fail(e, "merge launch");
  }
  return EID_OK;
}

int32_t eid_attn_decode(const eid_attn_desc *desc, const eid_attn_args *args, void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_attn_desc(desc)) return rc;
  if (desc->max_q_len != 1 || desc->num_q_tokens != desc->num_seqs)
    return fail(EID_ERR_INVALID_ARG, "decode needs max_q_len == 1 and num_q_tokens == num_seqs");
  if (int32_t rc = check_attn_args(desc, args, true, false)) return rc;
  return decode_launch(desc, args, hip_stream, false);
}

int32_t eid_attn_decode_noalloc(const eid_attn_desc *desc, const eid_attn_args *args,
                                void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_attn_desc(desc)) return rc;
  if (desc->max_q_len != 1 || desc->num_q_tokens != desc->num_seqs)
    return fail(EID_ERR_INVALID_ARG, "decode needs max_q_len == 1 and num_q_tokens == num_seqs");
  if (int32_t rc = check_attn_args(desc, args, true, false, false)) return rc;
  const Plan pl = make_plan(desc);
  const size_t need = eid::kPlanBytes + pl.parts_bytes + pl.ml_bytes + pl.acc_bytes;
  if (need > eid::kStaticScratchBytes)
    return fail(EID_ERR_WORKSPACE,
                "this batch needs %zu bytes of split-KV workspace; the library's static array holds "
                "%zu: use eid_attn_decode with a workspace of the caller's",
                need, (size_t)eid::kStaticScratchBytes);
  uint8_t *ws = nullptr;
  const hipError_t e = eid::static_scratch(&ws);
  if (e != hipSuccess) return hip_fail(e, "address of the static workspace");
  eid_attn_args own = *args;
  own.workspace = ws;
  own.workspace_bytes = eid::kStaticScratchBytes;
  // EID_DEBUG: every caller on a GPU shares the one array, and calls that overlap in time race
  // on it.  The checking mode remembers, per device, the stream of the last call and an event
  // recorded behind it, and refuses a call from another stream while that event is pending.
  // (Creates an event per device on first use: the checking mode does allocate.)
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const bool watch = debug_checks_on() && !stream_is_capturing(st);
  static std::mutex guard_mu;
  struct Guard { hipEvent_t done = nullptr; hipStream_t last = nullptr; bool used = false; };
  static Guard guards[64];
  int dev = 0;
  if (watch) {
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(EID_ERR_HIP, "EID_DEBUG: no current device");
    std::lock_guard<std::mutex> lock(guard_mu);
    Guard &g = guards[dev];
    if (g.used && g.last != st && hipEventQuery(g.done) == hipErrorNotReady)
      return fail(EID_ERR_INVALID_ARG,
                  "EID_DEBUG: eid_attn_decode_noalloc on one stream while a call on another stream is "
                  "still using the static workspace of this GPU");
    (void)hipGetLastError();
  }
  const int32_t rc = decode_launch(desc, &own, hip_stream, true);
  if (watch && rc == EID_OK) {
    std::lock_guard<std::mutex> lock(guard_mu);
    Guard &g = guards[dev];
    if (!g.done && hipEventCreateWithFlags(&g.done, hipEventDisableTiming) != hipSuccess) {
      g.done = nullptr;
      return hip_fail(hipGetLastError(), "EID_DEBUG: event for the static workspace");
    }
    if (hipEventRecord(g.done, st) != hipSuccess) return hip_fail(hipGetLastError(), "EID_DEBUG: event record");
    g.last = st;
    g.used = true;
  }
  return rc;
}

int32_t eid_attn_varlen(const eid_attn_desc *desc, const eid_attn_args *args, void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_attn_desc(desc)) return rc;
  if (int32_t rc = check_attn_args(desc, args, true, true)) return rc;
  if (args->k_new || args->v_new)
    return fail(EID_ERR_INVALID_ARG, "k_new / v_new are taken by eid_attn_decode only");
  const Plan pl = make_plan(desc);
  eid::AttnParams p = make_params(desc, args, pl);
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  const bool fp8 = desc->kv_dtype == EID_KV_FP8_E4M3;
  hipError_t e;
  // The kernels sort sequences into classes by q_len on the device.  When every sequence
  // has max_q_len query rows (num_q_tokens says so) the host knows the one class that is
  // populated and launches nothing for the others.
  const bool uniform = (int64_t)desc->num_seqs * desc->max_q_len == desc->num_q_tokens;
  const bool capturing = stream_is_capturing(st);
  if (debug_checks_on() && !capturing)
    if (int32_t rc = debug_check_host_copies(desc, args, false, st)) return rc;
  const int32_t qmax = short_q_max(desc);
  const bool only_verify = uniform && desc->max_q_len > 2 && desc->max_q_len <= qmax;
  const bool only_prefill = uniform && desc->max_q_len > qmax;
  int32_t *plan_slots = static_cast<int32_t *>(args->workspace);
  eid::EvenTable etab;  // (4 KiB)
  auto launch_split = [&](const ClassPlan &cp, const int ntiles, int32_t *slot) {
    if (cp.even) return eid::launch_even(p, ntiles, fp8, slot, st, &etab);
    if (!cp.short_span) return eid::launch_splitkv(p, ntiles, fp8, slot, st);
    p.plan = nullptr;  // the short-span kernel works with the host's partition
    p.plan_slot = slot;  // ... and records it for a merge called by itself afterwards
    const hipError_t es = eid::launch_shortspan(p, ntiles, fp8, st);
    p.plan_slot = nullptr;  // (the merge of this call takes p.partition)
    return es;
  };
  // Mixed batch: the MFMA-bound prefill launch and the HBM-bound split-KV launches use
  // different halves of the machine, so they run side by side: prefill on the thread's
  // helper stream, forked from and joined back into the caller's stream.
  const bool has_prefill = desc->max_q_len > qmax;
  static const bool serial = getenv("EID_SERIAL_CLASSES") != nullptr;  // for A/B measurements
  Helper *hs = (has_prefill && !only_prefill && !serial) ? helper_stream() : nullptr;
  // Two ways to run the classes on two streams.  fp8 cache (and EID_MIXED=share): the split-KV
  // kernels are held to one register-staged workgroup per CU and a prefill workgroup runs
  // beside it.  bf16 cache: the split-KV kernels stream through 128 KiB of LDS per CU, which
  // leaves no room for a prefill workgroup on the same CU, so the two classes share the device
  // by CUs: the even split of the split-KV rows is launched first with one workgroup for every
  // second CU (half the CUs move 5.4 TB/s of the 6.2 TB/s that all of them do), the prefill
  // workgroups fill the other CUs, and take over the rest as the split-KV workgroups end.
  // Config 3: 272 us, against 309 us one class after the other and 342 us side by side on
  // every CU.  EID_MIXED_DECODE_WGS sets the number of split-KV workgroups for measurements.
  static const bool share_env = [] {
    const char *m = getenv("EID_MIXED");
    return m && !strcmp(m, "share");
  }();
  const bool share = hs && (fp8 || share_env);
  static const int split_cus = [] {
    const char *m = getenv("EID_MIXED_DECODE_WGS");
    return m ? atoi(m) : 0;
  }();
  p.share_cus = share ? 1 : 0;
  p.mixed_wgs = (hs && !share) ? (split_cus > 0 ? split_cus : std::max(1, eid::device_cus() / 2)) : 0;
  p.fp8_pair = fp8_pair_applies(desc) ? 1 : 0;
  HelperJoin joiner;
  if (hs) {
    e = hipEventRecord(hs->fork, st);
    if (e == hipSuccess) e = hipStreamWaitEvent(hs->stream, hs->fork, 0);
    if (e != hipSuccess) return hip_fail(e, "fork to the helper stream");
    joiner.hs = hs;
    joiner.st = st;
    joiner.forked = true;
  }
  // With the host's copies of the lengths the prefill launch gets its query tiles listed,
  // heaviest first (not under capture: a captured launch serves whatever lengths a replay finds)
  eid::PfTable pf_tab;
  pf_tab.n = 0;
  auto list_tiles = [&](const eid::AttnParams &q) {
    if (args->seq_lens_host && args->cu_seqlens_q_host && !capturing)
      eid::build_prefill_table(q, args->seq_lens_host, args->cu_seqlens_q_host, &pf_tab);
  };
  auto prefill_on_helper = [&]() {
    eid::AttnParams pp = p;
    pp.qlen_lo = qmax + 1;
    pp.qlen_hi = 0x7fffffff;
    list_tiles(pp);
    return eid::launch_prefill(pp, desc->num_q_tokens, fp8, hs->stream, &pf_tab);
  };
  // q_len 1..2: one 16-row tile per KV head; each split-KV launch is followed by the merge
  // of its own class of sequences (they share the partition plan)
  ClassPlan cp1;
  cp1.skip = true;
  if (!only_verify && !only_prefill) {
    cp1 = plan_class(desc, args, pl, p, 1, 1, 2, false, &etab, nullptr, false, capturing);
    if (!cp1.skip) {
      e = launch_split(cp1, 1, plan_slots);
      if (e != hipSuccess) return hip_fail(e, "split-KV launch");
    }
  }
  if (hs) {  // the prefill rows, enqueued right behind the first split-KV launch
    e = prefill_on_helper();
    if (e != hipSuccess) return hip_fail(e, "prefill launch on the helper stream");
  }
  if (args->split_done_event) {
    e = hipEventRecord(static_cast<hipEvent_t>(args->split_done_event), st);
    if (e != hipSuccess) return hip_fail(e, "split_done_event record");
  }
  if (!cp1.skip && cp1.merge) {
    e = eid::launch_merge(p, st);
    if (e != hipSuccess) return hip_fail(e, "merge launch");
  }
  if (desc->max_q_len > 2 && !only_prefill) {  // q_len 3..6: three tiles
    const int vt = verify_tiles(desc);
    const ClassPlan cp3 = plan_class(desc, args, pl, p, vt, 3, qmax, false, &etab, nullptr, false, capturing);
    if (!cp3.skip) {
      e = launch_split(cp3, vt, plan_slots + 2);
      if (e != hipSuccess) return hip_fail(e, "split-KV (verify) launch");
      if (cp3.merge) {
        e = eid::launch_merge(p, st);
        if (e != hipSuccess) return hip_fail(e, "merge launch");
      }
    }
  }
  if (hs) {
    e = joiner.join();
    if (e != hipSuccess) return hip_fail(e, "join of the helper stream");
  } else if (has_prefill) {  // long chunks: MFMA prefill kernel
    p.qlen_lo = qmax + 1;
    p.qlen_hi = 0x7fffffff;
    list_tiles(p);
    e = eid::launch_prefill(p, desc->num_q_tokens, fp8, st, &pf_tab);
    if (e != hipSuccess) return hip_fail(e, "prefill launch");
  }
  return EID_OK;
}

int32_t eid_lse_merge(const eid_attn_desc *desc, const eid_attn_args *args, void *hip_stream) {
  g_err[0] = 0;
  if (int32_t rc = check_attn_desc(desc)) return rc;
  if (int32_t rc = check_attn_args(desc, args, false, false)) return rc;
  const Plan pl = make_plan(desc);
  eid::AttnParams p = make_params(desc, args, pl);
  // One class of sequences per call, as the split-KV launches are: q_len <= 2, else 3..6 (3..8).
  const bool fp8 = desc->kv_dtype == EID_KV_FP8_E4M3;
  p.qlen_lo = desc->max_q_len <= 2 ? 1 : 3;
  p.qlen_hi = desc->max_q_len <= 2 ? 2 : short_q_max(desc);
  p.target_items = eid::splitkv_fill(desc->max_q_len <= 2 ? 1 : verify_tiles(desc), fp8, desc->num_kv_heads);
  // With a run-time partition the merge takes the size the split-KV launch of this class
  // recorded in the workspace header (the attention entry points do the same).
  if (pl.dynamic)
    p.plan_slot = static_cast<int32_t *>(args->workspace) + (desc->max_q_len <= 2 ? 0 : 2);
  hipError_t e = eid::launch_merge(p, static_cast<hipStream_t>(hip_stream));
  if (e != hipSuccess) return hip_fail(e, "merge launch");
  return EID_OK;
}

int32_t eid_o_proj(const void *attn_out, const void *weight, const void *bias,
                   const void *residual, void *out, int32_t num_tokens, int32_t out_features,
                   int32_t in_features, void *hip_stream) {
  g_err[0] = 0;
  if (num_tokens < 0) return fail(EID_ERR_INVALID_ARG, "num_tokens %d < 0", num_tokens);
  if (in_features <= 0 || in_features % 64 != 0)
    return fail(EID_ERR_UNSUPPORTED, "in_features %d must be a positive multiple of 64", in_features);
  if (out_features <= 0 || out_features % 16 != 0)
    return fail(EID_ERR_UNSUPPORTED, "out_features %d must be a positive multiple of 16", out_features);
  if ((int64_t)num_tokens * out_features > (int64_t)0x7fffffff * 64 ||
      (int64_t)out_features * in_features > (int64_t)0x7fffffff * 64)
    return fail(EID_ERR_UNSUPPORTED, "matrix too large");
  if (num_tokens == 0) return EID_OK;
  if (!attn_out || !weight || !out)
    return fail(EID_ERR_INVALID_ARG, "attn_out, weight and out must be non-NULL");
  if (!aligned16(attn_out) || !aligned16(weight) || !aligned16(out) || !aligned16(bias) ||
      !aligned16(residual))
    return fail(EID_ERR_INVALID_ARG, "attn_out, weight, bias, residual and out must be 16-byte aligned");
  if (out == attn_out) return fail(EID_ERR_INVALID_ARG, "out must not alias attn_out");
  hipError_t e = eid::launch_o_proj(
      static_cast<const uint16_t *>(attn_out), static_cast<const uint16_t *>(weight),
      static_cast<const uint16_t *>(bias), static_cast<const uint16_t *>(residual),
      static_cast<uint16_t *>(out), num_tokens, out_features, in_features,
      static_cast<hipStream_t>(hip_stream));
  if (e != hipSuccess) return hip_fail(e, "o_proj launch");
  return EID_OK;
}

}  // extern "C"
