"""Operator-level host API over the C ABI: tensors in, status-checked launches out.

Every function takes torch tensors that already live on the GPU, checks dtype/shape/
contiguity on the host, and passes raw device pointers plus the current HIP stream to the
library.  Nothing here computes attention: if the HIP library is absent the call raises.
"""
import ctypes as C
import math
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib
from ._lib import AttnArgs, AttnDesc, KV_BF16, KV_FP8_E4M3, check, load_library


@dataclass
class AttnGeometry:
    """Static shape of one attention layer and its paged KV cache."""
    num_q_heads: int = 64
    num_kv_heads: int = 8
    head_dim: int = 64
    block_size: int = 16
    softmax_scale: float = 0.125
    window: int = 0          # 0 = full causal
    kv_dtype: int = KV_BF16
    partition_size: int = 0  # 0 = library picks


def make_desc(geom, *, num_seqs, num_q_tokens, max_q_len, max_kv_len, max_blocks_per_seq,
              num_blocks, sum_kv_len=0):
    d = AttnDesc()
    d.struct_size = C.sizeof(AttnDesc)
    d.num_seqs = num_seqs
    d.num_q_tokens = num_q_tokens
    d.max_q_len = max_q_len
    d.max_kv_len = max_kv_len
    d.num_q_heads = geom.num_q_heads
    d.num_kv_heads = geom.num_kv_heads
    d.head_dim = geom.head_dim
    d.block_size = geom.block_size
    d.max_blocks_per_seq = max_blocks_per_seq
    d.num_blocks = num_blocks
    d.softmax_scale = geom.softmax_scale
    d.window = geom.window
    d.kv_dtype = geom.kv_dtype
    d.partition_size = geom.partition_size
    d.sum_kv_len = sum_kv_len  # host-side sum of seq_lens (or an upper bound), 0 = unknown
    return d


def workspace_bytes(desc):
    return load_library().eid_workspace_bytes(C.byref(desc))


def partition_size(desc):
    return load_library().eid_partition_size(C.byref(desc))


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _kv_torch_dtype(kv_dtype):
    return torch.bfloat16 if kv_dtype == KV_BF16 else torch.uint8


def _require(t, name, dtype, ndim=None):
    if t is None:
        raise ValueError(f"{name} is None")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got {t.dim()}")


def _cache_view(t, geom, name):
    """Accept fp8 caches as uint8 or torch.float8_e4m3fn storage."""
    if geom.kv_dtype == KV_FP8_E4M3 and t.dtype == torch.float8_e4m3fn:
        t = t.view(torch.uint8)
    _require(t, name, _kv_torch_dtype(geom.kv_dtype), 4)
    if tuple(t.shape[1:]) != (geom.block_size, geom.num_kv_heads, geom.head_dim):
        raise ValueError(f"{name} must be [num_blocks, {geom.block_size}, {geom.num_kv_heads}, "
                         f"{geom.head_dim}], got {tuple(t.shape)}")
    return t


def kv_write(geom, k_new, v_new, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None):
    """Stage K1: cache_flat[slot_mapping[t]] = k_new[t] (bit copy, or fp8 quantise)."""
    _require(k_new, "k_new", torch.bfloat16, 3)
    _require(v_new, "v_new", torch.bfloat16, 3)
    k_cache = _cache_view(k_cache, geom, "k_cache")
    v_cache = _cache_view(v_cache, geom, "v_cache")
    _require(slot_mapping, "slot_mapping", torch.int64, 1)
    T = k_new.shape[0]
    if tuple(k_new.shape) != (T, geom.num_kv_heads, geom.head_dim) or k_new.shape != v_new.shape:
        raise ValueError("k_new / v_new must be [T, num_kv_heads, head_dim]")
    if slot_mapping.shape[0] != T:
        raise ValueError("slot_mapping must have one entry per new token")
    if k_cache.shape != v_cache.shape:
        raise ValueError("k_cache and v_cache shapes differ")
    if geom.kv_dtype == KV_FP8_E4M3:
        _require(k_scale, "k_scale", torch.float32, 1)
        _require(v_scale, "v_scale", torch.float32, 1)
    desc = make_desc(geom, num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                     max_blocks_per_seq=1, num_blocks=k_cache.shape[0])
    check(load_library().eid_kv_write(C.byref(desc), _ptr(k_new), _ptr(v_new), _ptr(k_cache),
                                      _ptr(v_cache), _ptr(slot_mapping), T, _ptr(k_scale),
                                      _ptr(v_scale), _stream()))


def rope_kv_write(geom, qkv, positions, cos_sin, k_cache, v_cache, slot_mapping, k_scale=None,
                  v_scale=None, q_out=None):
    """Fused RoPE + QKV split + slot-mapped KV write.  qkv is [T, (Hq + 2 Hkv) * D] bf16,
    cos_sin [max_pos, D] fp32 (per position D/2 cosines then D/2 sines); returns q_out
    [T, Hq, D] bf16."""
    _require(qkv, "qkv", torch.bfloat16, 2)
    _require(positions, "positions", torch.int32, 1)
    _require(cos_sin, "cos_sin", torch.float32, 2)
    k_cache = _cache_view(k_cache, geom, "k_cache")
    v_cache = _cache_view(v_cache, geom, "v_cache")
    _require(slot_mapping, "slot_mapping", torch.int64, 1)
    T = qkv.shape[0]
    if qkv.shape[1] != (geom.num_q_heads + 2 * geom.num_kv_heads) * geom.head_dim:
        raise ValueError("qkv must be [T, (num_q_heads + 2 num_kv_heads) * head_dim]")
    if positions.shape[0] != T or slot_mapping.shape[0] != T:
        raise ValueError("positions and slot_mapping must have one entry per token")
    if cos_sin.shape[1] != geom.head_dim:
        raise ValueError("cos_sin must be [max_pos, head_dim]")
    if geom.kv_dtype == KV_FP8_E4M3:
        _require(k_scale, "k_scale", torch.float32, 1)
        _require(v_scale, "v_scale", torch.float32, 1)
    if q_out is None:
        q_out = torch.empty((T, geom.num_q_heads, geom.head_dim), dtype=torch.bfloat16,
                            device=qkv.device)
    else:
        _require(q_out, "q_out", torch.bfloat16, 3)
    desc = make_desc(geom, num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                     max_blocks_per_seq=1, num_blocks=k_cache.shape[0])
    check(load_library().eid_rope_kv_write(
        C.byref(desc), _ptr(qkv), _ptr(positions), _ptr(cos_sin), cos_sin.shape[0], _ptr(q_out),
        _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), T, _ptr(k_scale), _ptr(v_scale),
        _stream()))
    return q_out


def qkv_rope_kv_write(geom, hidden, weight, bias, positions, cos_sin, k_cache, v_cache,
                      slot_mapping, k_scale=None, v_scale=None, q_out=None):
    """QKV projection + rope_kv_write in one launch (at most 64 tokens): hidden [T, K] bf16,
    weight [(Hq + 2 Hkv) * D, K] bf16, bias [(Hq + 2 Hkv) * D] bf16 or None; the rest as
    rope_kv_write.  Returns q_out [T, Hq, D] bf16; bit-identical to o_proj + rope_kv_write."""
    _require(hidden, "hidden", torch.bfloat16, 2)
    _require(weight, "weight", torch.bfloat16, 2)
    _require(positions, "positions", torch.int32, 1)
    _require(cos_sin, "cos_sin", torch.float32, 2)
    k_cache = _cache_view(k_cache, geom, "k_cache")
    v_cache = _cache_view(v_cache, geom, "v_cache")
    _require(slot_mapping, "slot_mapping", torch.int64, 1)
    T, K = hidden.shape
    N = (geom.num_q_heads + 2 * geom.num_kv_heads) * geom.head_dim
    if tuple(weight.shape) != (N, K):
        raise ValueError(f"weight must be [{N}, {K}]")
    if bias is not None:
        _require(bias, "bias", torch.bfloat16, 1)
        if bias.shape[0] != N:
            raise ValueError(f"bias must be [{N}]")
    if positions.shape[0] != T or slot_mapping.shape[0] != T:
        raise ValueError("positions and slot_mapping must have one entry per token")
    if cos_sin.shape[1] != geom.head_dim:
        raise ValueError("cos_sin must be [max_pos, head_dim]")
    if geom.kv_dtype == KV_FP8_E4M3:
        _require(k_scale, "k_scale", torch.float32, 1)
        _require(v_scale, "v_scale", torch.float32, 1)
    if q_out is None:
        q_out = torch.empty((T, geom.num_q_heads, geom.head_dim), dtype=torch.bfloat16,
                            device=hidden.device)
    else:
        _require(q_out, "q_out", torch.bfloat16, 3)
    desc = make_desc(geom, num_seqs=1, num_q_tokens=1, max_q_len=1, max_kv_len=1,
                     max_blocks_per_seq=1, num_blocks=k_cache.shape[0])
    check(load_library().eid_qkv_rope_kv_write(
        C.byref(desc), _ptr(hidden), _ptr(weight), _ptr(bias), K, _ptr(positions), _ptr(cos_sin),
        cos_sin.shape[0], _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), T,
        _ptr(k_scale), _ptr(v_scale), _stream()))
    return q_out


def o_proj(attn_out, weight, bias=None, residual=None, out=None):
    """Output projection after attention: attn_out [T, Hq, D] (or [T, K]) bf16, weight [N, K]
    bf16 (out_features x in_features), optional bias [N] and residual [T, N] bf16; returns
    out [T, N] bf16 = attn_out @ weight^T + bias + residual (fp32 sums, one bf16 rounding).
    `out` may be the residual buffer itself."""
    if attn_out.dim() == 3:
        attn_out = attn_out.reshape(attn_out.shape[0], -1)
    _require(attn_out, "attn_out", torch.bfloat16, 2)
    _require(weight, "weight", torch.bfloat16, 2)
    T, K = attn_out.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise ValueError("weight must be [out_features, in_features] with in_features = %d" % K)
    if bias is not None:
        _require(bias, "bias", torch.bfloat16, 1)
        if bias.shape[0] != N:
            raise ValueError("bias must be [out_features]")
    if residual is not None:
        _require(residual, "residual", torch.bfloat16, 2)
        if tuple(residual.shape) != (T, N):
            raise ValueError("residual must be [T, out_features]")
    if out is None:
        out = torch.empty((T, N), dtype=torch.bfloat16, device=attn_out.device)
    else:
        _require(out, "out", torch.bfloat16, 2)
        if tuple(out.shape) != (T, N):
            raise ValueError("out must be [T, out_features]")
    check(load_library().eid_o_proj(_ptr(attn_out), _ptr(weight), _ptr(bias), _ptr(residual),
                                    _ptr(out), T, N, K, _stream()))
    return out


def yarn_cos_sin(max_pos, head_dim=64, base=150000.0, scaling_factor=32.0,
                 initial_context=4096.0, ntk_alpha=1.0, ntk_beta=32.0):
    """[max_pos, head_dim] fp32 table for eid_rope_kv_write (numpy): per position head_dim/2
    cosines then head_dim/2 sines with YaRN "NTK-by-parts" frequency blending and the
    attention-temperature factor 0.1 ln(scaling_factor) + 1 folded in, as the published
    gpt-oss model definition describes its rotary embedding (defaults are that model's
    configuration).  scaling_factor <= 1 gives plain RoPE."""
    half = head_dim // 2
    freq = base ** (np.arange(0, head_dim, 2, dtype=np.float64) / head_dim)
    if scaling_factor > 1.0:
        concentration = 0.1 * np.log(scaling_factor) + 1.0
        low = half * np.log(initial_context / (ntk_beta * 2 * np.pi)) / np.log(base)
        high = half * np.log(initial_context / (ntk_alpha * 2 * np.pi)) / np.log(base)
        ramp = (np.arange(half, dtype=np.float64) - low) / (high - low)
        mask = 1.0 - np.clip(ramp, 0.0, 1.0)
        inv_freq = (1.0 / (scaling_factor * freq)) * (1.0 - mask) + (1.0 / freq) * mask
    else:
        concentration = 1.0
        inv_freq = 1.0 / freq
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv_freq[None, :]
    return np.concatenate([np.cos(ang) * concentration, np.sin(ang) * concentration],
                          axis=1).astype(np.float32)


def _host_i32(a, name, n):
    """A host copy of a length array as contiguous int32 numpy (the library reads it during
    the call); accepts numpy arrays and CPU tensors."""
    if a is None:
        return None
    if isinstance(a, torch.Tensor):
        if a.is_cuda:
            raise ValueError(f"{name} must live in host memory")
        a = a.numpy()
    a = np.ascontiguousarray(a, dtype=np.int32)
    if a.shape != (n,):
        raise ValueError(f"{name} must have {n} entries")
    return a


def _host_bt(a, block_table):
    """A host copy of the block table as contiguous int32 numpy of the device table's shape."""
    if a is None:
        return None
    if isinstance(a, torch.Tensor):
        if a.is_cuda:
            raise ValueError("block_table_host must live in host memory")
        a = a.numpy()
    a = np.ascontiguousarray(a, dtype=np.int32)
    if a.shape != tuple(block_table.shape):
        raise ValueError("block_table_host must have the shape of block_table")
    return a


def _attn_call(fn_name, geom, q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q,
               max_q_len, max_kv_len, sinks, k_scale, v_scale, out, lse, workspace,
               return_lse, sum_kv_len=0, k_new=None, v_new=None, seq_lens_host=None,
               cu_seqlens_q_host=None, block_table_host=None):
    _require(q, "q", torch.bfloat16, 3)
    k_cache = _cache_view(k_cache, geom, "k_cache")
    v_cache = _cache_view(v_cache, geom, "v_cache")
    _require(block_table, "block_table", torch.int32, 2)
    _require(seq_lens, "seq_lens", torch.int32, 1)
    S = seq_lens.shape[0]
    T = q.shape[0]
    if tuple(q.shape[1:]) != (geom.num_q_heads, geom.head_dim):
        raise ValueError("q must be [T, num_q_heads, head_dim]")
    if block_table.shape[0] != S:
        raise ValueError("block_table must have one row per sequence")
    if cu_seqlens_q is not None:
        _require(cu_seqlens_q, "cu_seqlens_q", torch.int32, 1)
        if cu_seqlens_q.shape[0] != S + 1:
            raise ValueError("cu_seqlens_q must have num_seqs + 1 entries")
    if sinks is not None:
        _require(sinks, "sinks", torch.float32, 1)
    if geom.kv_dtype == KV_FP8_E4M3:
        _require(k_scale, "k_scale", torch.float32, 1)
        _require(v_scale, "v_scale", torch.float32, 1)
    desc = make_desc(geom, num_seqs=S, num_q_tokens=T, max_q_len=max_q_len,
                     max_kv_len=max_kv_len, max_blocks_per_seq=block_table.shape[1],
                     num_blocks=k_cache.shape[0], sum_kv_len=sum_kv_len)
    if out is None:
        out = torch.empty_like(q)
    else:
        _require(out, "out", torch.bfloat16, 3)
    if return_lse and lse is None:
        lse = torch.empty((T, geom.num_q_heads), dtype=torch.float32, device=q.device)
    lib = load_library()
    need = lib.eid_workspace_bytes(C.byref(desc))
    if need == 0:
        check(getattr(lib, fn_name)(C.byref(desc), C.byref(AttnArgs()), None))
    own_ws = fn_name == "eid_attn_decode_noalloc"   # the library's static array serves it
    if workspace is None and not own_ws:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    args = AttnArgs()
    args.q = q.data_ptr()
    args.out = out.data_ptr()
    args.lse = lse.data_ptr() if lse is not None else None
    args.k_cache = k_cache.data_ptr()
    args.v_cache = v_cache.data_ptr()
    args.block_table = block_table.data_ptr()
    args.cu_seqlens_q = cu_seqlens_q.data_ptr() if cu_seqlens_q is not None else None
    args.seq_lens = seq_lens.data_ptr()
    args.sinks = sinks.data_ptr() if sinks is not None else None
    args.k_scale = k_scale.data_ptr() if k_scale is not None else None
    args.v_scale = v_scale.data_ptr() if v_scale is not None else None
    if not own_ws:
        args.workspace = workspace.data_ptr()
        args.workspace_bytes = workspace.numel() * workspace.element_size()
    for name, t in (("k_new", k_new), ("v_new", v_new)):
        if t is not None:
            _require(t, name, torch.bfloat16, 3)
            if tuple(t.shape) != (S, geom.num_kv_heads, geom.head_dim):
                raise ValueError(f"{name} must be [num_seqs, num_kv_heads, head_dim]")
            setattr(args, name, t.data_ptr())
    sl_h = _host_i32(seq_lens_host, "seq_lens_host", S)
    cu_h = _host_i32(cu_seqlens_q_host, "cu_seqlens_q_host", S + 1)
    args.seq_lens_host = sl_h.ctypes.data if sl_h is not None else None
    args.cu_seqlens_q_host = cu_h.ctypes.data if cu_h is not None else None
    bt_h = _host_bt(block_table_host, block_table)
    args.block_table_host = bt_h.ctypes.data if bt_h is not None else None
    check(getattr(lib, fn_name)(C.byref(desc), C.byref(args), _stream()))
    return (out, lse) if return_lse else out


class PreparedCall:
    """A validated (desc, args) pair bound to one entry point: calling it only crosses the
    C ABI (no tensor checks, no allocation), for launch-rate-sensitive loops.  The tensors
    are kept alive by the object."""

    def __init__(self, fn_name, desc, args, keep, out, lse):
        self._fn = getattr(load_library(), fn_name)
        self.desc, self.args, self._keep, self.out, self.lse = desc, args, keep, out, lse
        self._d, self._a = C.byref(desc), C.byref(args)

    def __call__(self, stream=None):
        st = _stream() if stream is None else C.c_void_p(stream)
        rc = self._fn(self._d, self._a, st)
        if rc:
            check(rc)
        return self.out

    def bound_to(self, lib):
        """The same call through another build of the library (the measurement build)."""
        other = PreparedCall.__new__(PreparedCall)
        other.__dict__.update(self.__dict__)
        other._fn = getattr(lib, self._fn.__name__)
        return other


def prepare(fn_name, geom, q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q=None, *,
            max_q_len=1, max_kv_len, sinks=None, k_scale=None, v_scale=None, out=None, lse=None,
            workspace=None, sum_kv_len=0, k_new=None, v_new=None, seq_lens_host=None,
            cu_seqlens_q_host=None, block_table_host=None):
    """Build a PreparedCall for "eid_attn_decode" / "eid_attn_varlen" / "eid_lse_merge".
    `seq_lens_host` / `cu_seqlens_q_host` (host copies of the two length arrays) are copied
    and kept by the object."""
    k_cache = _cache_view(k_cache, geom, "k_cache")
    v_cache = _cache_view(v_cache, geom, "v_cache")
    _require(q, "q", torch.bfloat16, 3)
    _require(block_table, "block_table", torch.int32, 2)
    _require(seq_lens, "seq_lens", torch.int32, 1)
    desc = make_desc(geom, num_seqs=seq_lens.shape[0], num_q_tokens=q.shape[0],
                     max_q_len=max_q_len, max_kv_len=max_kv_len,
                     max_blocks_per_seq=block_table.shape[1], num_blocks=k_cache.shape[0],
                     sum_kv_len=sum_kv_len)
    need = load_library().eid_workspace_bytes(C.byref(desc))
    if need == 0:
        check(getattr(load_library(), fn_name)(C.byref(desc), C.byref(AttnArgs()), None))
    if out is None:
        out = torch.empty_like(q)
    own_ws = fn_name == "eid_attn_decode_noalloc"   # the library's static array serves it
    if workspace is None and not own_ws:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    args = AttnArgs()
    args.q, args.out = q.data_ptr(), out.data_ptr()
    args.lse = lse.data_ptr() if lse is not None else None
    args.k_cache, args.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
    args.block_table, args.seq_lens = block_table.data_ptr(), seq_lens.data_ptr()
    args.cu_seqlens_q = cu_seqlens_q.data_ptr() if cu_seqlens_q is not None else None
    args.sinks = sinks.data_ptr() if sinks is not None else None
    args.k_scale = k_scale.data_ptr() if k_scale is not None else None
    args.v_scale = v_scale.data_ptr() if v_scale is not None else None
    if not own_ws:
        args.workspace = workspace.data_ptr()
        args.workspace_bytes = workspace.numel()
    args.k_new = k_new.data_ptr() if k_new is not None else None
    args.v_new = v_new.data_ptr() if v_new is not None else None
    S = seq_lens.shape[0]
    sl_h = _host_i32(seq_lens_host, "seq_lens_host", S)
    cu_h = _host_i32(cu_seqlens_q_host, "cu_seqlens_q_host", S + 1)
    sl_h = sl_h.copy() if sl_h is not None else None
    cu_h = cu_h.copy() if cu_h is not None else None
    args.seq_lens_host = sl_h.ctypes.data if sl_h is not None else None
    args.cu_seqlens_q_host = cu_h.ctypes.data if cu_h is not None else None
    bt_h = _host_bt(block_table_host, block_table)
    bt_h = bt_h.copy() if bt_h is not None else None
    args.block_table_host = bt_h.ctypes.data if bt_h is not None else None
    keep = (q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q, sinks, k_scale, v_scale,
            k_new, v_new, sl_h, cu_h, bt_h,
            workspace)  # workspace stays last: callers share it via _keep[-1]
    return PreparedCall(fn_name, desc, args, keep, out, lse)


def attn_decode(geom, q, k_cache, v_cache, block_table, seq_lens, *, max_kv_len, sinks=None,
                k_scale=None, v_scale=None, out=None, lse=None, workspace=None,
                return_lse=False, sum_kv_len=0, k_new=None, v_new=None, seq_lens_host=None,
                block_table_host=None):
    """Stages K2+K4: one query row per sequence (q is [num_seqs, Hq, D]).  `sum_kv_len` is the
    optional host-side sum of seq_lens (any upper bound): it sizes the launch to the work;
    `seq_lens_host`, a host copy of seq_lens, lets the library plan the launch exactly.
    With `k_new` / `v_new` ([num_seqs, Hkv, D] bf16: the newest token of every sequence, not
    yet in the cache) the call writes those rows into the caches itself (stage K1 fused)."""
    return _attn_call("eid_attn_decode", geom, q, k_cache, v_cache, block_table, seq_lens, None,
                      1, max_kv_len, sinks, k_scale, v_scale, out, lse, workspace, return_lse,
                      sum_kv_len, k_new, v_new, seq_lens_host, None, block_table_host)


def attn_decode_noalloc(geom, q, k_cache, v_cache, block_table, seq_lens, *, max_kv_len, out,
                        sinks=None, k_scale=None, v_scale=None, lse=None, sum_kv_len=0,
                        k_new=None, v_new=None, seq_lens_host=None, block_table_host=None):
    """attn_decode through the entry point that allocates nothing: the split-KV partials go
    to the library's static device array (batches whose workspace would exceed
    STATIC_WORKSPACE_BYTES raise EID_ERR_WORKSPACE), and `out` must be given.  Calls on one
    GPU share that array and must not overlap in time."""
    if out is None:
        raise ValueError("out must be given: this call allocates nothing")
    return _attn_call("eid_attn_decode_noalloc", geom, q, k_cache, v_cache, block_table,
                      seq_lens, None, 1, max_kv_len, sinks, k_scale, v_scale, out, lse, None,
                      False, sum_kv_len, k_new, v_new, seq_lens_host, None, block_table_host)


def attn_varlen(geom, q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q, *, max_q_len,
                max_kv_len, sinks=None, k_scale=None, v_scale=None, out=None, lse=None,
                workspace=None, return_lse=False, sum_kv_len=0, seq_lens_host=None,
                cu_seqlens_q_host=None):
    """Stages K2/K3+K4 on a ragged cu_seqlens batch (prefill chunks, verify rows, decodes).
    With host copies of both length arrays the library plans the launches exactly."""
    return _attn_call("eid_attn_varlen", geom, q, k_cache, v_cache, block_table, seq_lens,
                      cu_seqlens_q, max_q_len, max_kv_len, sinks, k_scale, v_scale, out, lse,
                      workspace, return_lse, sum_kv_len, None, None, seq_lens_host,
                      cu_seqlens_q_host)


def lse_merge(geom, workspace, seq_lens, cu_seqlens_q, *, num_q_tokens, max_q_len, max_kv_len,
              max_blocks_per_seq, num_blocks, sinks=None, out=None, lse=None):
    """Stage K4 alone over partials already present in `workspace` (see workspace_layout)."""
    S = seq_lens.shape[0]
    desc = make_desc(geom, num_seqs=S, num_q_tokens=num_q_tokens, max_q_len=max_q_len,
                     max_kv_len=max_kv_len, max_blocks_per_seq=max_blocks_per_seq,
                     num_blocks=num_blocks)
    if out is None:
        out = torch.zeros((num_q_tokens, geom.num_q_heads, geom.head_dim), dtype=torch.bfloat16,
                          device=workspace.device)
    args = AttnArgs()
    args.out = out.data_ptr()
    args.lse = lse.data_ptr() if lse is not None else None
    args.cu_seqlens_q = cu_seqlens_q.data_ptr() if cu_seqlens_q is not None else None
    args.seq_lens = seq_lens.data_ptr()
    args.sinks = sinks.data_ptr() if sinks is not None else None
    args.workspace = workspace.data_ptr()
    args.workspace_bytes = workspace.numel() * workspace.element_size()
    check(load_library().eid_lse_merge(C.byref(desc), C.byref(args), _stream()))
    return out


def workspace_layout(desc):
    """(partition, nparts_max, ws_rows, ml_offset, acc_offset): after a 256-byte plan header
    (and, when a sequence can have more than one partition, one int32 per sequence: its number
    of pieces) the split-KV workspace holds
    ml  float32 [num_seqs*ws_rows, nparts_max, Hq, 2]  (m in natural-log units, l) and
    o   float16 [num_seqs*ws_rows, nparts_max, Hq, 64] (partition output sum e^(s-m) v / l) at
    the byte offsets returned."""
    P = partition_size(desc)
    if (16 < desc.max_q_len <= 32 and desc.num_kv_heads % 8 == 0
            and desc.num_seqs * desc.num_kv_heads <= 64):
        qmax = 32
    elif (8 < desc.max_q_len <= 16 and desc.num_kv_heads % 8 == 0
            and desc.num_seqs * desc.num_kv_heads <= 448):
        qmax = 16   # rows of a split-KV sequence (see short_q_max in eid_api.cpp)
    else:
        qmax = 8 if 6 < desc.max_q_len <= 8 else 6
    if desc.window > 0:
        span = min(desc.max_kv_len, desc.window + qmax + desc.block_size - 1)
    else:
        span = desc.max_kv_len
    nparts = (span + P - 1) // P
    head = 256
    if nparts > 1:
        # (see make_plan in eid_api.cpp) the per-sequence piece counts of an even split sit behind
        # the plan header; with a run-time partition the ranges are cut anywhere in a sequence:
        # one more piece than whole partitions
        if desc.partition_size == 0 and P == 256:
            nparts += 1
        head += (desc.num_seqs * 4 + 255) // 256 * 256
    ws_rows = min(desc.max_q_len, qmax)
    cells = desc.num_seqs * ws_rows * desc.num_q_heads * nparts
    ml_bytes = (cells * 8 + 255) // 256 * 256
    return P, nparts, ws_rows, head, head + ml_bytes
