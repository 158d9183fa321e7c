"""Host tests of the block allocator / batch-metadata builder (include/eidola_sched.h).
No GPU needed: the scheduler is host code.  Besides direct checks of every array, a random
schedule of add / build / free operations is replayed against an independent pure-Python
model of the same policy and every output is compared exactly."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import eidola_amd as ea
from eidola_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BS = 16


def test_header_and_library_agree_on_the_scheduler_symbols():
    header = open(os.path.join(ROOT, "include", "eidola_sched.h")).read()
    declared = set(re.findall(r"\b(eid_sched_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.SCHED_EXPORTS)
    lib = ea.load_library()
    for name in declared:
        assert hasattr(lib, name), name
    assert C.sizeof(_lib.SchedConfig) == 24 and C.sizeof(_lib.BatchInfo) == 24


def test_one_step_layout():
    s = ea.Scheduler(num_blocks=32, max_blocks_per_seq=8)
    for i in (7, 8, 9):
        assert s.add_seq(i) == 0
    b = s.build_batch([7, 8, 9], [20, 1, 16])
    assert (b.num_seqs, b.num_q_tokens, b.max_q_len, b.max_kv_len, b.sum_kv_len) == (3, 37, 20, 20, 37)
    assert b.cu_seqlens_q.tolist() == [0, 20, 21, 37]
    assert b.seq_lens.tolist() == [20, 1, 16]
    assert b.positions.tolist() == list(range(20)) + [0] + list(range(16))
    # blocks are handed out in pool order: seq 7 -> 0,1; seq 8 -> 2; seq 9 -> 3
    assert b.block_table[0, :2].tolist() == [0, 1] and b.block_table[1, 0] == 2 and b.block_table[2, 0] == 3
    assert b.slot_mapping.tolist() == list(range(20)) + [32] + list(range(48, 64))
    assert s.free_blocks == 28
    # decode step: one token each, seq 9 crosses into a new block
    d = s.build_batch([9, 7, 8], [1, 1, 1])
    assert d.seq_lens.tolist() == [17, 21, 2] and d.positions.tolist() == [16, 20, 1]
    assert d.block_table[0, :2].tolist() == [3, 4]
    assert d.slot_mapping.tolist() == [4 * BS, 1 * BS + 4, 2 * BS + 1]
    assert d.sum_kv_len == 40 and d.max_kv_len == 21 and s.free_blocks == 27
    assert s.seq_len(7) == 21 and s.seq_len(12345) == -1


def test_exhaustion_changes_nothing():
    s = ea.Scheduler(num_blocks=4, max_blocks_per_seq=4)
    s.add_seq(1)
    s.add_seq(2)
    s.build_batch([1], [30])                     # 2 blocks
    with pytest.raises(ea.EidError) as e:
        s.build_batch([1, 2], [3, 33])           # needs 1 + 3 > 2 free
    assert e.value.name == "EID_ERR_NO_BLOCKS"
    assert s.free_blocks == 2 and s.seq_len(1) == 30 and s.seq_len(2) == 0
    b = s.build_batch([1, 2], [3, 16])           # 1 + 1 fits
    assert b.seq_lens.tolist() == [33, 16] and s.free_blocks == 0
    s.free_seq(1)
    assert s.free_blocks == 3
    assert [s.block_refs(i) for i in range(4)] == [0, 0, 0, 1]


def test_invalid_requests():
    with pytest.raises(ea.EidError):
        ea.Scheduler(num_blocks=0, max_blocks_per_seq=4)
    with pytest.raises(ea.EidError):
        ea.Scheduler(num_blocks=8, max_blocks_per_seq=4, block_size=32)
    s = ea.Scheduler(num_blocks=8, max_blocks_per_seq=2)
    s.add_seq(1)
    with pytest.raises(ea.EidError):
        s.add_seq(1)
    with pytest.raises(ea.EidError):
        s.build_batch([2], [1])                  # unknown sequence
    with pytest.raises(ea.EidError):
        s.build_batch([1, 1], [1, 1])            # listed twice
    with pytest.raises(ea.EidError):
        s.build_batch([1], [0])
    with pytest.raises(ea.EidError) as e:
        s.build_batch([1], [33])                 # 3 blocks > max_blocks_per_seq
    assert e.value.name == "EID_ERR_INVALID_ARG" and s.seq_len(1) == 0 and s.free_blocks == 8
    with pytest.raises(ea.EidError):
        s.free_seq(5)


def test_prefix_reuse_shares_full_blocks_and_leaves_a_token_to_compute():
    s = ea.Scheduler(num_blocks=16, max_blocks_per_seq=8, prefix_reuse=True)
    prompt = np.arange(100, 148)                 # 48 tokens = 3 full blocks
    assert s.add_seq(1, prompt) == 0
    s.build_batch([1], [48], prompt)
    # same prompt: only two blocks are taken, the last token block is left to compute
    assert s.add_seq(2, prompt) == 32
    b = s.build_batch([2], [16], prompt[32:])
    assert b.block_table[0, :3].tolist() == [0, 1, 3] and b.positions.tolist() == list(range(32, 48))
    assert [s.block_refs(i) for i in range(4)] == [2, 2, 1, 1]
    # a prompt that diverges inside the second block shares only the first
    other = prompt.copy()
    other[20] = -5
    assert s.add_seq(3, other) == 16
    # longer prompt with the same 48-token head: all three indexed blocks match
    assert s.add_seq(4, np.concatenate([prompt, [1, 2, 3]])) == 48
    assert s.block_refs(2) == 2                  # seq 1's third block, not seq 2's copy
    # no tokens given for a step: that sequence stops being indexed, nothing breaks
    s.build_batch([3], [20])
    assert s.add_seq(5, other[:40]) == 16


def test_freed_prefix_is_found_again_and_tails_are_recycled_first():
    s = ea.Scheduler(num_blocks=6, max_blocks_per_seq=6, prefix_reuse=True)
    p = np.arange(64)
    s.add_seq(1, p)
    s.build_batch([1], [64], p)                  # blocks 0..3, all indexed
    s.free_seq(1)
    assert s.free_blocks == 6
    # free list is now 4,5 (never used) then 3,2,1,0: a 3-block allocation takes 4,5,3
    s.add_seq(2)
    b = s.build_batch([2], [48])
    assert b.block_table[0, :3].tolist() == [4, 5, 3]
    # the head of the old prefix (blocks 0,1,2) is still matchable; block 3 is gone
    assert s.add_seq(3, np.arange(80)) == 48
    assert [s.block_refs(i) for i in range(6)] == [1, 1, 1, 1, 1, 1] and s.free_blocks == 0


class Model:
    """Independent restatement of the policy: LRU free list (oldest first), allocation pops
    the head and forgets that block's index entry, blocks of a freed sequence are queued last
    block first, full blocks are indexed by their whole token prefix (first copy wins)."""

    def __init__(self, n, mb, reuse):
        self.free = list(range(n))
        self.refs = [0] * n
        self.key_of = {}           # block -> prefix tuple it is indexed under
        self.index = {}            # prefix tuple -> block
        self.seqs = {}
        self.mb, self.reuse = mb, reuse

    def alloc(self):
        b = self.free.pop(0)
        k = self.key_of.pop(b, None)
        if k is not None and self.index.get(k) == b:
            del self.index[k]
        self.refs[b] = 1
        return b

    def add(self, sid, prompt):
        blocks, toks = [], []
        if self.reuse and prompt is not None and len(prompt) > 1:
            for i in range(min((len(prompt) - 1) // BS, self.mb)):
                key = tuple(prompt[: (i + 1) * BS])
                b = self.index.get(key)
                if b is None:
                    break
                if self.refs[b] == 0:
                    self.free.remove(b)
                self.refs[b] += 1
                blocks.append(b)
                toks = list(key)
        self.seqs[sid] = dict(blocks=blocks, toks=toks, len=len(toks), chained=True)
        return len(toks)

    def free_seq(self, sid):
        for b in reversed(self.seqs.pop(sid)["blocks"]):
            self.refs[b] -= 1
            if self.refs[b] == 0:
                self.free.append(b)

    def build(self, ids, qls, new):
        need = sum(-(-(self.seqs[i]["len"] + q) // BS) - len(self.seqs[i]["blocks"]) for i, q in zip(ids, qls))
        if need > len(self.free):
            return None
        slots, pos, sl, rows = [], [], [], []
        r = 0
        for i, q in zip(ids, qls):
            s = self.seqs[i]
            if self.reuse and new is None:
                s["chained"] = False
            for _ in range(q):
                p = s["len"]
                if p % BS == 0:
                    s["blocks"].append(self.alloc())
                b = s["blocks"][p // BS]
                slots.append(b * BS + p % BS)
                pos.append(p)
                if self.reuse and new is not None and s["chained"]:
                    s["toks"].append(int(new[r]))
                    if len(s["toks"]) % BS == 0:
                        key = tuple(s["toks"])
                        if key not in self.index:
                            self.index[key] = b
                            self.key_of[b] = key
                s["len"] += 1
                r += 1
            sl.append(s["len"])
            rows.append(list(s["blocks"]))
        return slots, pos, sl, rows


@pytest.mark.parametrize("reuse", [False, True])
def test_random_schedule_matches_the_python_model(reuse):
    rng = np.random.default_rng(11 if reuse else 12)
    N, MB = 48, 10
    s, m = ea.Scheduler(N, MB, prefix_reuse=reuse), Model(N, MB, reuse)
    heads = [rng.integers(0, 50, size=64) for _ in range(3)]   # shared prompt heads
    live, pending, next_id = [], {}, 0
    for step in range(400):
        op = rng.random()
        if op < 0.25 and len(live) < 8:
            prompt = np.concatenate([heads[rng.integers(3)][: rng.integers(1, 65)],
                                     rng.integers(0, 50, size=rng.integers(0, 30))]).astype(np.int32)
            cached = s.add_seq(next_id, prompt)
            assert cached == m.add(next_id, prompt)
            live.append(next_id)
            pending[next_id] = list(prompt[cached:])
            next_id += 1
        elif op < 0.35 and live:
            sid = live.pop(rng.integers(len(live)))
            pending.pop(sid)
            s.free_seq(sid)
            m.free_seq(sid)
        elif live:
            k = rng.integers(1, len(live) + 1)
            ids = [int(x) for x in rng.permutation(live)[:k]]
            qls, toks = [], []
            for sid in ids:
                left = pending[sid]
                q = int(rng.integers(1, min(len(left), 24) + 1)) if left else 1
                new = left[:q] if left else [int(rng.integers(0, 50))]
                qls.append(q)
                toks += new
            with_tokens = rng.random() < 0.9
            exp = m.build(ids, qls, toks if with_tokens else None) if all(
                -(-(m.seqs[i]["len"] + q) // BS) <= MB for i, q in zip(ids, qls)) else "too long"
            if exp == "too long" or exp is None:
                with pytest.raises(ea.EidError):
                    s.build_batch(ids, qls, toks if with_tokens else None)
                if exp is None:
                    assert s.free_blocks == len(m.free)
                continue
            b = s.build_batch(ids, qls, toks if with_tokens else None)
            for sid, q in zip(ids, qls):
                pending[sid] = pending[sid][q:]
            slots, pos, sl, rows = exp
            assert b.slot_mapping.tolist() == slots and b.positions.tolist() == pos
            assert b.seq_lens.tolist() == sl and b.sum_kv_len == sum(sl) and b.max_kv_len == max(sl)
            for r, row in enumerate(rows):
                assert b.block_table[r, : len(row)].tolist() == row
        assert s.free_blocks == len(m.free)
        assert [s.block_refs(i) for i in range(N)] == m.refs
        # conservation: every block is free or referenced
        assert s.free_blocks + sum(1 for r in m.refs if r > 0) == N
