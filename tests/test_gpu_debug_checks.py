"""EID_DEBUG=1: the attention entry points verify what they otherwise take on trust: host
copies of seq_lens / block_table equal the device arrays, desc.sum_kv_len is not below the
true sum, eid_kv_write's slots are distinct.  The switch is read once per process, so the
checks run in a child process that has it set from the start."""
import os
import subprocess
import sys
import textwrap

import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = textwrap.dedent("""
    import sys, os
    sys.path.insert(0, os.path.join(%r, "tests")); sys.path.insert(0, %r)
    import numpy as np, torch
    import eidola_amd as ea
    import gpu_helpers as G
    from helpers import make_batch, logical_tensors
    b = make_batch([700, 33, 2500, 129], [1, 1, 1, 1])
    q, k, v, sinks = logical_tensors(b)
    kc_d, vc_d = G.gpu_caches(b, k, v)
    args = (b.geom, G.bf16_dev(q), kc_d, vc_d, G.dev(b.block_table), G.dev(b.seq_lens))
    kw = dict(max_kv_len=b.max_kv_len, sinks=G.dev(sinks))
    good = ea.attn_decode(*args, sum_kv_len=int(b.seq_lens.sum()), seq_lens_host=b.seq_lens,
                          block_table_host=b.block_table, **kw)
    torch.cuda.synchronize()
    def refused(what, **extra):
        try:
            ea.attn_decode(*args, **{**kw, **extra})
        except ea.EidError as e:
            assert e.name == "EID_ERR_INVALID_ARG" and "EID_DEBUG" in str(e) and what in str(e), str(e)
            return
        raise AssertionError("accepted: " + what)
    wrong = b.seq_lens.copy(); wrong[2] -= 1
    refused("seq_lens_host", seq_lens_host=wrong)
    refused("sum_kv_len", sum_kv_len=int(b.seq_lens.sum()) - 1)
    bt = b.block_table.copy(); bt[0, 3] += 1
    refused("block_table_host", seq_lens_host=b.seq_lens, block_table_host=bt)
    # entries past a sequence's last page are never compared
    bt = b.block_table.copy(); bt[1, 40] = 123456
    ea.attn_decode(*args, seq_lens_host=b.seq_lens, block_table_host=bt, **kw)
    # duplicate slots
    kn = torch.zeros((3, 8, 64), dtype=torch.bfloat16, device="cuda:0")
    try:
        ea.kv_write(b.geom, kn, kn, kc_d, vc_d, G.dev(np.array([5, -1, 5], dtype=np.int64)))
    except ea.EidError as e:
        assert "more than once" in str(e), str(e)
    else:
        raise AssertionError("duplicate slots accepted")
    ea.kv_write(b.geom, kn, kn, kc_d, vc_d, G.dev(np.array([5, -1, -1], dtype=np.int64)))
    torch.cuda.synchronize()
    print("debug checks ok")
""") % (ROOT, ROOT)


def test_debug_mode_catches_mismatched_host_copies_and_duplicate_slots():
    assert torch.cuda.is_available()
    env = dict(os.environ, EID_DEBUG="1")
    r = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "debug checks ok" in r.stdout, r.stdout + r.stderr


CHILD_NOALLOC = textwrap.dedent("""
    import sys, os
    sys.path.insert(0, %r)
    import torch
    import eidola_amd as ea
    # 16 sequences of 120,000 tokens: the call's kernels run for most of a millisecond, far longer
    # than the host needs to reach the next call (the checking mode waits for the stream before
    # every launch, so only the last call's kernels can still be running)
    S, L = 16, 120000
    pages = S * (L // 16)
    geom = ea.AttnGeometry(partition_size=2048)
    gen = torch.Generator(device="cuda:0").manual_seed(1)
    kc = torch.randn((pages, 16, 8, 64), generator=gen, device="cuda:0", dtype=torch.bfloat16)
    vc = torch.randn((pages, 16, 8, 64), generator=gen, device="cuda:0", dtype=torch.bfloat16)
    q = torch.randn((S, 64, 64), generator=gen, device="cuda:0", dtype=torch.bfloat16)
    bt = torch.arange(pages, device="cuda:0", dtype=torch.int32).view(S, L // 16).contiguous()
    sl = torch.full((S,), L, device="cuda:0", dtype=torch.int32)
    args = (geom, q, kc, vc, bt, sl)
    out, out2 = torch.zeros_like(q), torch.zeros_like(q)
    torch.cuda.synchronize()
    one, two = torch.cuda.Stream(), torch.cuda.Stream()
    # (first uses take milliseconds: the library's one-time set-up, a stream's hardware queue)
    with torch.cuda.stream(one):
        ea.attn_decode_noalloc(*args, max_kv_len=L, out=out)
    with torch.cuda.stream(two):
        torch.zeros(8, device="cuda:0").add_(1)
    torch.cuda.synchronize()
    with torch.cuda.stream(one):
        ea.attn_decode_noalloc(*args, max_kv_len=L, out=out)
    with torch.cuda.stream(two):
        try:
            ea.attn_decode_noalloc(*args, max_kv_len=L, out=out2)
        except ea.EidError as e:
            assert e.name == "EID_ERR_INVALID_ARG" and "static workspace" in str(e), str(e)
        else:
            raise AssertionError("overlapping use of the static workspace accepted")
    torch.cuda.synchronize()
    with torch.cuda.stream(two):   # the first stream has drained: the other one may have the array
        ea.attn_decode_noalloc(*args, max_kv_len=L, out=out2)
    with torch.cuda.stream(two):   # and again on the same stream, back to back: one stream orders its calls
        ea.attn_decode_noalloc(*args, max_kv_len=L, out=out2)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    print("static workspace guard ok")
""") % (ROOT,)


def test_debug_mode_refuses_overlapping_calls_on_the_static_workspace():
    assert torch.cuda.is_available()
    env = dict(os.environ, EID_DEBUG="1")
    r = subprocess.run([sys.executable, "-c", CHILD_NOALLOC], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "static workspace guard ok" in r.stdout, r.stdout + r.stderr
