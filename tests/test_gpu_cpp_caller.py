"""The C ABI driven from C++ alone (tests/cpp/abi_caller.cpp, built by tests/cpp/Makefile):
eid_kv_write + eid_attn_decode in a process without Python or torch, its output against the
fp64 oracle and the written cache rows bit for bit."""
import os
import subprocess

import numpy as np
import pytest

from eidola_amd import synth
from helpers import assert_close, cpu_caches, logical_tensors, make_batch, oracle_out

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "abi_caller")


@pytest.mark.parametrize("window", [0, 128])
def test_cpp_caller_kv_write_and_decode(tmp_path, window):
    assert os.path.exists(EXE), "tests/cpp/abi_caller is not built: make -C tests/cpp (build() does)"
    b = make_batch([37, 128, 511, 1000, 2300], [1, 1, 1, 1, 1], window=window)
    q, k, v, sinks = logical_tensors(b)
    kc, vc = cpu_caches(b, k, v)
    ref, _ = oracle_out(b, q, kc, vc, sinks)
    # the newest token of every sequence is what the caller writes: take it out of the caches
    slots = b.slot_mapping.astype(np.int64)
    flat_k, flat_v = kc.reshape(-1, 8, 64), vc.reshape(-1, 8, 64)
    k_new, v_new = flat_k[slots].copy(), flat_v[slots].copy()
    flat_k[slots] = 0x7FC1
    flat_v[slots] = 0x7FC1
    inp, outp = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(inp, "wb") as f:
        np.array([b.num_seqs, b.block_table.shape[1], b.num_blocks, window, b.max_kv_len], np.int32).tofile(f)
        for a in (q, k_new, v_new, kc, vc, b.block_table.astype(np.int32), b.seq_lens.astype(np.int32),
                  slots, sinks.astype(np.float32)):
            np.ascontiguousarray(a).tofile(f)
    r = subprocess.run([EXE, str(inp), str(outp)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    got = np.fromfile(outp, dtype=np.uint16)
    n_out, n_row = b.num_seqs * 64 * 64, b.num_seqs * 8 * 64
    assert got.size == n_out + 2 * n_row
    assert_close(got[:n_out].reshape(b.num_seqs, 64, 64), ref, f"C++ caller, window {window}")
    assert np.array_equal(got[n_out:n_out + n_row].reshape(-1, 8, 64), k_new)
    assert np.array_equal(got[n_out + n_row:].reshape(-1, 8, 64), v_new)
