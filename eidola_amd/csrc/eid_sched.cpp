// Paged-KV block allocator and batch-metadata builder (host code only; see
// include/eidola_sched.h for the contract).  Data structures:
//   blocks_   per physical block: reference count, links of the free list, and (prefix reuse)
//             the chained hash, the parent's hash and the 16 token ids it was indexed with
//   free list doubly linked through the blocks, oldest-freed at the head; allocation pops the
//             head, which evicts that block's index entry if it still has one
//   index_    hash -> block of every indexed full block, referenced or free
//   seqs_     per sequence: block list, length, hash of its last indexed block, and the token
//             ids of its partly filled last block (they are hashed when the block fills)
#include <cstdarg>
#include <cstdint>
#include <algorithm>
#include <cstring>
#include <new>
#include <unordered_map>
#include <vector>

#include "../../include/eidola_attn.h"
#include "../../include/eidola_sched.h"

namespace eid {
int32_t set_error(int32_t status, const char *fmt, va_list ap);
void clear_error();
}  // namespace eid

namespace {

int32_t fail(eid_status st, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  const int32_t rc = eid::set_error((int32_t)st, fmt, ap);
  va_end(ap);
  return rc;
}

inline uint64_t mix64(uint64_t z) {  // SplitMix64 finaliser
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

constexpr uint64_t kRootHash = 0x5EED0F5EED0F5EEDull;  // parent hash of a sequence's first block

uint64_t block_hash(uint64_t parent, const int32_t *tokens, int n) {
  uint64_t h = mix64(parent);
  for (int i = 0; i < n; ++i) h = mix64(h ^ (uint64_t)(uint32_t)tokens[i]);
  return h;
}

struct Block {
  int32_t refs = 0;
  bool indexed = false;    // present in index_ under `hash`
  int64_t prev = -1, next = -1;  // free-list links (meaningful while refs == 0)
  uint64_t hash = 0, parent = 0;
};

struct Seq {
  std::vector<int64_t> blocks;
  int32_t len = 0;
  uint64_t chain = kRootHash;  // hash of the last full block while `chained`
  bool chained = true;         // every full block so far has been hashed
  std::vector<int32_t> tail;   // token ids of the partly filled last block
  uint64_t stamp = 0;          // eid_sched::stamp of the last build_batch call that listed it
};

}  // namespace

struct eid_sched {
  int32_t bs = 16;
  int64_t nblocks = 0;
  int32_t max_blocks_per_seq = 0;
  bool reuse = false;
  std::vector<Block> blocks;
  std::vector<int32_t> block_tokens;  // [nblocks][bs], prefix reuse only
  int64_t free_head = -1, free_tail = -1, free_count = 0;
  uint64_t stamp = 0;  // build_batch call counter
  std::unordered_map<uint64_t, int64_t> index;
  std::unordered_map<int64_t, Seq> seqs;

  void free_push_back(int64_t b) {
    Block &B = blocks[b];
    B.prev = free_tail;
    B.next = -1;
    if (free_tail >= 0) blocks[free_tail].next = b; else free_head = b;
    free_tail = b;
    ++free_count;
  }
  void free_unlink(int64_t b) {
    Block &B = blocks[b];
    if (B.prev >= 0) blocks[B.prev].next = B.next; else free_head = B.next;
    if (B.next >= 0) blocks[B.next].prev = B.prev; else free_tail = B.prev;
    B.prev = B.next = -1;
    --free_count;
  }
  // Oldest free block; whatever prefix it still indexed is forgotten.
  int64_t allocate() {
    const int64_t b = free_head;
    free_unlink(b);
    Block &B = blocks[b];
    if (B.indexed) {
      auto it = index.find(B.hash);
      if (it != index.end() && it->second == b) index.erase(it);
      B.indexed = false;
    }
    B.refs = 1;
    return b;
  }
  void release(int64_t b) {
    Block &B = blocks[b];
    if (--B.refs == 0) free_push_back(b);
  }
  // Block indexed under (parent, tokens), or -1.
  int64_t lookup(uint64_t parent, const int32_t *tokens, uint64_t h) const {
    auto it = index.find(h);
    if (it == index.end()) return -1;
    const int64_t b = it->second;
    const Block &B = blocks[b];
    if (!B.indexed || B.hash != h || B.parent != parent) return -1;
    if (std::memcmp(&block_tokens[(size_t)b * bs], tokens, sizeof(int32_t) * bs) != 0) return -1;
    return b;
  }
};

extern "C" {

int32_t eid_sched_create(const eid_sched_config *cfg, eid_sched **out) {
  eid::clear_error();
  if (!cfg || !out) return fail(EID_ERR_INVALID_ARG, "cfg and out must be non-NULL");
  *out = nullptr;
  if (cfg->struct_size != sizeof(eid_sched_config))
    return fail(EID_ERR_INVALID_ARG, "cfg.struct_size %u != %zu", cfg->struct_size,
                sizeof(eid_sched_config));
  if (cfg->block_size != 16) return fail(EID_ERR_UNSUPPORTED, "block_size %d unsupported (16 only)", cfg->block_size);
  if (cfg->num_blocks <= 0 || cfg->num_blocks > (int64_t)0x7fffffff)
    return fail(EID_ERR_INVALID_ARG, "num_blocks %lld out of range", (long long)cfg->num_blocks);
  if (cfg->max_blocks_per_seq <= 0) return fail(EID_ERR_INVALID_ARG, "max_blocks_per_seq must be positive");
  eid_sched *s = new (std::nothrow) eid_sched;
  if (!s) return fail(EID_ERR_INVALID_ARG, "out of host memory");
  try {  // no C++ exception may cross the C ABI
    s->bs = cfg->block_size;
    s->nblocks = cfg->num_blocks;
    s->max_blocks_per_seq = cfg->max_blocks_per_seq;
    s->reuse = cfg->prefix_reuse != 0;
    s->blocks.resize((size_t)s->nblocks);
    if (s->reuse) s->block_tokens.assign((size_t)s->nblocks * s->bs, 0);
  } catch (...) {
    delete s;
    return fail(EID_ERR_INVALID_ARG, "out of host memory for %lld blocks", (long long)cfg->num_blocks);
  }
  for (int64_t b = 0; b < s->nblocks; ++b) s->free_push_back(b);
  *out = s;
  return EID_OK;
}

void eid_sched_destroy(eid_sched *s) { delete s; }

int32_t eid_sched_add_seq(eid_sched *s, int64_t seq_id, const int32_t *prompt, int32_t n,
                          int32_t *cached_tokens) {
  eid::clear_error();
  if (!s) return fail(EID_ERR_INVALID_ARG, "scheduler is NULL");
  if (n < 0) return fail(EID_ERR_INVALID_ARG, "prompt length %d is negative", n);
  if (s->seqs.count(seq_id)) return fail(EID_ERR_INVALID_ARG, "sequence %lld already exists", (long long)seq_id);
  Seq q;
  try {  // every allocation happens before the first block reference is taken
    q.blocks.reserve((size_t)std::min<int64_t>(s->max_blocks_per_seq, (int64_t)n / s->bs + 1));
    q.tail.reserve((size_t)s->bs);
  } catch (...) {
    return fail(EID_ERR_INVALID_ARG, "out of host memory");
  }
  if (s->reuse && prompt && n > 1) {
    const int max_match = (n - 1) / s->bs;  // at least one token stays to be computed
    for (int b = 0; b < max_match && b < s->max_blocks_per_seq; ++b) {
      const int32_t *tok = prompt + (size_t)b * s->bs;
      const uint64_t h = block_hash(q.chain, tok, s->bs);
      const int64_t hit = s->lookup(q.chain, tok, h);
      if (hit < 0) break;
      Block &B = s->blocks[hit];
      if (B.refs == 0) s->free_unlink(hit);
      ++B.refs;
      q.blocks.push_back(hit);
      q.chain = h;
      q.len += s->bs;
    }
  }
  const int32_t cached = q.len;
  std::vector<int64_t> taken;
  try {
    taken = q.blocks;
    s->seqs.emplace(seq_id, std::move(q));
  } catch (...) {  // give the references back: the call changes nothing when it fails
    const std::vector<int64_t> &held = taken.empty() ? q.blocks : taken;
    for (size_t i = held.size(); i-- > 0;) s->release(held[i]);
    return fail(EID_ERR_INVALID_ARG, "out of host memory");
  }
  if (cached_tokens) *cached_tokens = cached;
  return EID_OK;
}

int32_t eid_sched_free_seq(eid_sched *s, int64_t seq_id) {
  eid::clear_error();
  if (!s) return fail(EID_ERR_INVALID_ARG, "scheduler is NULL");
  auto it = s->seqs.find(seq_id);
  if (it == s->seqs.end()) return fail(EID_ERR_INVALID_ARG, "sequence %lld unknown", (long long)seq_id);
  // last block first: the free list hands out its oldest entries first, so the tail of a
  // prefix chain is recycled before its head and the head stays matchable for longer
  for (size_t i = it->second.blocks.size(); i-- > 0;) s->release(it->second.blocks[i]);
  s->seqs.erase(it);
  return EID_OK;
}

int32_t eid_sched_seq_len(const eid_sched *s, int64_t seq_id) {
  if (!s) return -1;
  auto it = s->seqs.find(seq_id);
  return it == s->seqs.end() ? -1 : it->second.len;
}

int64_t eid_sched_free_blocks(const eid_sched *s) { return s ? s->free_count : -1; }

int32_t eid_sched_block_refs(const eid_sched *s, int64_t block) {
  if (!s || block < 0 || block >= s->nblocks) return -1;
  return s->blocks[(size_t)block].refs;
}

int32_t eid_sched_build_batch(eid_sched *s, const int64_t *seq_ids, const int32_t *q_lens,
                              int32_t num_seqs, const int32_t *new_tokens,
                              int32_t *block_table, int64_t *slot_mapping,
                              int32_t *cu_seqlens_q, int32_t *seq_lens, int32_t *positions,
                              eid_batch_info *info) {
  eid::clear_error();
  if (!s) return fail(EID_ERR_INVALID_ARG, "scheduler is NULL");
  if (num_seqs <= 0 || !seq_ids || !q_lens)
    return fail(EID_ERR_INVALID_ARG, "num_seqs must be positive, seq_ids and q_lens non-NULL");
  if (!block_table || !slot_mapping || !cu_seqlens_q || !seq_lens || !info)
    return fail(EID_ERR_INVALID_ARG, "output arrays and info must be non-NULL");
  const int bs = s->bs;
  // pass 1: validate, count the blocks the step needs; nothing is modified
  int64_t need = 0, total_q = 0;
  std::vector<Seq *> sq;
  try {
    sq.resize((size_t)num_seqs);
  } catch (...) {
    return fail(EID_ERR_INVALID_ARG, "out of host memory");
  }
  const uint64_t stamp = ++s->stamp;  // marks the sequences of this call: finds duplicates in O(1)
  for (int i = 0; i < num_seqs; ++i) {
    auto it = s->seqs.find(seq_ids[i]);
    if (it == s->seqs.end()) return fail(EID_ERR_INVALID_ARG, "sequence %lld unknown", (long long)seq_ids[i]);
    if (q_lens[i] < 1) return fail(EID_ERR_INVALID_ARG, "q_lens[%d] = %d must be >= 1", i, q_lens[i]);
    Seq *q = &it->second;
    if (q->stamp == stamp) return fail(EID_ERR_INVALID_ARG, "sequence %lld listed twice", (long long)seq_ids[i]);
    q->stamp = stamp;
    sq[(size_t)i] = q;
    const int64_t new_len = (int64_t)q->len + q_lens[i];
    const int64_t nb = (new_len + bs - 1) / bs;
    if (nb > s->max_blocks_per_seq)
      return fail(EID_ERR_INVALID_ARG, "sequence %lld would need %lld blocks (max_blocks_per_seq %d)",
                  (long long)seq_ids[i], (long long)nb, s->max_blocks_per_seq);
    need += nb - (int64_t)q->blocks.size();
    try {  // capacity only: pass 2 must not allocate, so it cannot fail half way
      q->blocks.reserve((size_t)nb);
      q->tail.reserve((size_t)bs);
    } catch (...) {
      return fail(EID_ERR_INVALID_ARG, "out of host memory");
    }
    total_q += q_lens[i];
    if (total_q > 0x7fffffff) return fail(EID_ERR_INVALID_ARG, "more than 2^31 query tokens");
  }
  if (need > s->free_count)
    return fail(EID_ERR_NO_BLOCKS, "step needs %lld new blocks, %lld are free", (long long)need,
                (long long)s->free_count);
  // pass 2: reserve and write
  int32_t row = 0, max_q = 0, max_kv = 0;
  int64_t sum_kv = 0;
  cu_seqlens_q[0] = 0;
  for (int i = 0; i < num_seqs; ++i) {
    Seq &q = *sq[(size_t)i];
    const int ql = q_lens[i];
    const bool hash_now = s->reuse && new_tokens && q.chained;
    if (s->reuse && !new_tokens) {  // tokens unknown: this sequence's chain ends here
      q.chained = false;
      q.tail.clear();
    }
    for (int t = 0; t < ql; ++t) {
      const int pos = q.len;
      if (pos % bs == 0) q.blocks.push_back(s->allocate());
      const int64_t blk = q.blocks[(size_t)(pos / bs)];
      slot_mapping[row] = blk * bs + pos % bs;
      if (positions) positions[row] = pos;
      if (hash_now) {
        q.tail.push_back(new_tokens[row]);
        if ((int)q.tail.size() == bs) {  // block full: index it
          const uint64_t h = block_hash(q.chain, q.tail.data(), bs);
          Block &B = s->blocks[(size_t)blk];
          B.hash = h;
          B.parent = q.chain;
          std::memcpy(&s->block_tokens[(size_t)blk * bs], q.tail.data(), sizeof(int32_t) * bs);
          try {
            if (s->index.emplace(h, blk).second) B.indexed = true;  // first copy of a prefix wins
          } catch (...) {
            // no memory for the index node: the block simply stays unshared
          }
          q.chain = h;
          q.tail.clear();
        }
      }
      ++q.len;
      ++row;
    }
    int32_t *bt = block_table + (size_t)i * s->max_blocks_per_seq;
    for (size_t b = 0; b < q.blocks.size(); ++b) bt[b] = (int32_t)q.blocks[b];
    cu_seqlens_q[i + 1] = row;
    seq_lens[i] = q.len;
    max_q = ql > max_q ? ql : max_q;
    max_kv = q.len > max_kv ? q.len : max_kv;
    sum_kv += q.len;
  }
  info->num_seqs = num_seqs;
  info->num_q_tokens = row;
  info->max_q_len = max_q;
  info->max_kv_len = max_kv;
  info->sum_kv_len = sum_kv;
  return EID_OK;
}

}  // extern "C"
