"""GPU-side plumbing for the parity tests: numpy bit arrays <-> torch device tensors."""
import numpy as np
import torch

import eidola_amd as ea
from eidola_amd import KV_FP8_E4M3, synth

from helpers import desc_of, empty_caches, all_slots

DEV = "cuda:0"


def bf16_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV).view(torch.bfloat16)


def bits_host(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def dev(a, dtype=None):
    if a is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def cache_dev(c):
    if c.dtype == np.uint8:
        return torch.from_numpy(c).to(DEV)
    return bf16_dev(c)


def cache_host(t):
    if t.dtype == torch.uint8:
        return t.cpu().numpy()
    return bits_host(t)


def gpu_caches(batch, k, v, k_scale=None, v_scale=None):
    """Poisoned device caches filled through eid_kv_write with every context token."""
    kc, vc = empty_caches(batch)
    kc_d, vc_d = cache_dev(kc), cache_dev(vc)
    ea.kv_write(batch.geom, bf16_dev(k), bf16_dev(v), kc_d, vc_d, dev(all_slots(batch)),
                dev(k_scale), dev(v_scale))
    return kc_d, vc_d


def run_attn(batch, q, kc_d, vc_d, sinks, k_scale=None, v_scale=None, *, decode=None,
             return_lse=False, geom=None, hint=False, return_device=False, host_lens=False):
    """Calls eid_attn_decode (all q_len == 1) or eid_attn_varlen through the C ABI; with
    `hint` the host-side sum of seq_lens is passed as desc.sum_kv_len, with `host_lens` the
    host copies of seq_lens / cu_seqlens_q as well.  `return_device` hands back the output
    tensor itself instead of its bits on the host."""
    geom = geom or batch.geom
    if decode is None:
        decode = batch.max_q_len == 1
    kw = dict(max_kv_len=batch.max_kv_len, sinks=dev(sinks), k_scale=dev(k_scale),
              v_scale=dev(v_scale), return_lse=return_lse,
              sum_kv_len=int(batch.seq_lens.sum()) if hint else 0)
    bt, sl = dev(batch.block_table), dev(batch.seq_lens)
    if host_lens:
        kw["seq_lens_host"] = batch.seq_lens
    if decode:
        if host_lens:
            kw["block_table_host"] = batch.block_table
        r = ea.attn_decode(geom, bf16_dev(q), kc_d, vc_d, bt, sl, **kw)
    else:
        if host_lens:
            kw["cu_seqlens_q_host"] = batch.cu_seqlens_q
        r = ea.attn_varlen(geom, bf16_dev(q), kc_d, vc_d, bt, sl, dev(batch.cu_seqlens_q),
                           max_q_len=batch.max_q_len, **kw)
    torch.cuda.synchronize()
    if return_device:
        return r[0] if return_lse else r
    if return_lse:
        return bits_host(r[0]), r[1].cpu().numpy()
    return bits_host(r)


def compact_to_cpu(batch, kc_d, vc_d, seqs):
    """Gather the pages of the chosen sequences into a small CPU cache; returns
    (sub-batch, k_cache_np, v_cache_np) with a remapped block table."""
    from dataclasses import replace
    seqs = list(seqs)
    nblk = (batch.seq_lens[seqs].astype(np.int64) + 15) // 16
    pages = np.concatenate([batch.block_table[s, :n] for s, n in zip(seqs, nblk)])
    idx = torch.from_numpy(pages.astype(np.int64)).to(kc_d.device)
    kc = cache_host(kc_d[idx])
    vc = cache_host(vc_d[idx])
    bt = np.zeros((len(seqs), int(nblk.max())), dtype=np.int32)
    off = 0
    for i, n in enumerate(nblk):
        bt[i, :n] = np.arange(off, off + n)
        off += int(n)
    sub = synth.Batch(batch.name + "_sub", batch.geom, batch.seq_lens[seqs], batch.q_lens[seqs],
                      bt, len(pages), batch.seed)
    return sub, kc, vc


def rows_of(batch, seqs):
    cu = batch.cu_seqlens_q
    return np.concatenate([np.arange(cu[s], cu[s + 1]) for s in seqs])
