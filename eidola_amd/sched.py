"""Host-side mirror of ``include/eidola_sched.h``: the paged-KV block allocator and
batch-metadata builder that turns a continuous-batching schedule into the arrays the
attention kernels take.  Pure host code (numpy buffers); the arithmetic is in
``eidola_amd/csrc/eid_sched.cpp``."""
import ctypes as C
from dataclasses import dataclass

import numpy as np

from ._lib import BatchInfo, SchedConfig, check, load_library


@dataclass
class BuiltBatch:
    """Arrays and scalars of one step, ready for kv_write / attn_decode / attn_varlen."""
    block_table: np.ndarray    # [num_seqs, max_blocks_per_seq] int32
    slot_mapping: np.ndarray   # [num_q_tokens] int64
    cu_seqlens_q: np.ndarray   # [num_seqs + 1] int32
    seq_lens: np.ndarray       # [num_seqs] int32
    positions: np.ndarray      # [num_q_tokens] int32
    num_seqs: int
    num_q_tokens: int
    max_q_len: int
    max_kv_len: int
    sum_kv_len: int


class Scheduler:
    def __init__(self, num_blocks, max_blocks_per_seq, *, block_size=16, prefix_reuse=False):
        self._h = None
        self._lib = load_library()
        cfg = SchedConfig(C.sizeof(SchedConfig), block_size, num_blocks, max_blocks_per_seq,
                          1 if prefix_reuse else 0)
        h = C.c_void_p()
        check(self._lib.eid_sched_create(C.byref(cfg), C.byref(h)))
        self._h = h
        self.num_blocks, self.max_blocks_per_seq, self.block_size = num_blocks, max_blocks_per_seq, block_size

    def close(self):
        if self._h:
            self._lib.eid_sched_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def add_seq(self, seq_id, prompt=None):
        """Registers a sequence; returns the number of prompt tokens already in the cache."""
        cached = C.c_int32(0)
        if prompt is None:
            check(self._lib.eid_sched_add_seq(self._h, seq_id, None, 0, C.byref(cached)))
        else:
            p = np.ascontiguousarray(prompt, dtype=np.int32)
            check(self._lib.eid_sched_add_seq(self._h, seq_id, p.ctypes.data, p.size, C.byref(cached)))
        return cached.value

    def free_seq(self, seq_id):
        check(self._lib.eid_sched_free_seq(self._h, seq_id))

    def seq_len(self, seq_id):
        return self._lib.eid_sched_seq_len(self._h, seq_id)

    @property
    def free_blocks(self):
        return self._lib.eid_sched_free_blocks(self._h)

    def block_refs(self, block):
        return self._lib.eid_sched_block_refs(self._h, block)

    def build_batch(self, seq_ids, q_lens, new_tokens=None, block_table=None):
        ids = np.ascontiguousarray(seq_ids, dtype=np.int64)
        ql = np.ascontiguousarray(q_lens, dtype=np.int32)
        if ids.shape != ql.shape or ids.ndim != 1:
            raise ValueError("seq_ids and q_lens must be 1-D and of equal length")
        S = ids.size
        T = int(ql.clip(min=0).sum())
        if block_table is None:
            block_table = np.zeros((S, self.max_blocks_per_seq), dtype=np.int32)
        slot = np.empty(T, dtype=np.int64)
        cu = np.empty(S + 1, dtype=np.int32)
        sl = np.empty(S, dtype=np.int32)
        pos = np.empty(T, dtype=np.int32)
        tok = None
        if new_tokens is not None:
            tok = np.ascontiguousarray(new_tokens, dtype=np.int32)
            if tok.size != T:
                raise ValueError("new_tokens must hold one id per new token")
        info = BatchInfo()
        check(self._lib.eid_sched_build_batch(
            self._h, ids.ctypes.data, ql.ctypes.data, S, tok.ctypes.data if tok is not None else None,
            block_table.ctypes.data, slot.ctypes.data, cu.ctypes.data, sl.ctypes.data,
            pos.ctypes.data, C.byref(info)))
        return BuiltBatch(block_table, slot, cu, sl, pos, info.num_seqs, info.num_q_tokens,
                          info.max_q_len, info.max_kv_len, info.sum_kv_len)
