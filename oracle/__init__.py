"""Python face of the CPU oracle (TEST INFRASTRUCTURE ONLY — see eid_oracle.h).

Importable from tests/, from __graft_entry__.smoke() and from bench.py's cpu_baseline leg,
never from the eidola_amd package.  `liboracle.so` is the C restatement; `oracle_np` is an
independently written numpy restatement used to cross-check it on small inputs.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from eidola_amd._lib import AttnArgs, AttnDesc

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        P = C.c_void_p
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_fp8_e4m3_encode.argtypes = [C.c_float]
        L.orc_fp8_e4m3_encode.restype = C.c_uint8
        L.orc_fp8_e4m3_decode.argtypes = [C.c_uint8]
        L.orc_fp8_e4m3_decode.restype = C.c_float
        L.orc_kv_write.argtypes = [C.POINTER(AttnDesc), P, P, P, P, P, C.c_int32, P, P]
        L.orc_kv_write.restype = C.c_int
        L.orc_rope_kv_write.argtypes = [C.POINTER(AttnDesc), P, P, P, C.c_int32, P, P, P, P,
                                        C.c_int32, P, P]
        L.orc_rope_kv_write.restype = C.c_int
        L.orc_o_proj.argtypes = [P, P, P, P, P, P, C.c_int32, C.c_int32, C.c_int32]
        L.orc_o_proj.restype = None
        L.orc_f64_to_bf16.argtypes = [C.c_double]
        L.orc_f64_to_bf16.restype = C.c_uint16
        L.orc_attn_f64.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnArgs), P, P]
        L.orc_attn_f64.restype = C.c_int
        L.orc_splitkv_partials_f64.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnArgs),
                                               C.c_int32, C.c_int32, P, P]
        L.orc_splitkv_partials_f64.restype = C.c_int
        L.orc_lse_merge_f64.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.c_int32, P, P, P, P, P]
        L.orc_lse_merge_f64.restype = C.c_int
        L.orc_kv_begin.argtypes = [C.c_int32] * 4
        L.orc_kv_begin.restype = C.c_int32
        L.orc_attn_bf16.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnArgs), C.c_int]
        L.orc_attn_bf16.restype = C.c_int
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _host_args(q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q, sinks, k_scale,
               v_scale, out=None, lse=None):
    keep = dict(
        q=_c(q, np.uint16), k=np.ascontiguousarray(k_cache), v=np.ascontiguousarray(v_cache),
        bt=_c(block_table, np.int32), sl=_c(seq_lens, np.int32), cu=_c(cu_seqlens_q, np.int32),
        sinks=_c(sinks, np.float32), ks=_c(k_scale, np.float32), vs=_c(v_scale, np.float32),
        out=out, lse=lse)
    a = AttnArgs()
    a.q = _p(keep["q"])
    a.out = _p(out)
    a.lse = _p(lse)
    a.k_cache = _p(keep["k"])
    a.v_cache = _p(keep["v"])
    a.block_table = _p(keep["bt"])
    a.cu_seqlens_q = _p(keep["cu"])
    a.seq_lens = _p(keep["sl"])
    a.sinks = _p(keep["sinks"])
    a.k_scale = _p(keep["ks"])
    a.v_scale = _p(keep["vs"])
    return a, keep


def kv_write(desc, k_new, v_new, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None):
    """In-place on the numpy caches (uint16 for bf16, uint8 for fp8)."""
    k_new = _c(k_new, np.uint16)
    v_new = _c(v_new, np.uint16)
    sm = _c(slot_mapping, np.int64)
    ks, vs = _c(k_scale, np.float32), _c(v_scale, np.float32)
    assert k_cache.flags.c_contiguous and v_cache.flags.c_contiguous
    rc = lib().orc_kv_write(C.byref(desc), _p(k_new), _p(v_new), _p(k_cache), _p(v_cache),
                            _p(sm), len(sm), _p(ks), _p(vs))
    if rc:
        raise ValueError("slot out of range")


def rope_kv_write(desc, qkv, positions, cos_sin, k_cache, v_cache, slot_mapping, k_scale=None,
                  v_scale=None):
    """Fused RoPE + split + KV write; caches are updated in place, q_out [T,Hq,D] (bf16 bits)
    is returned."""
    qkv = _c(qkv, np.uint16)
    pos = _c(positions, np.int32)
    cs = _c(cos_sin, np.float32)
    sm = _c(slot_mapping, np.int64)
    ks, vs = _c(k_scale, np.float32), _c(v_scale, np.float32)
    assert k_cache.flags.c_contiguous and v_cache.flags.c_contiguous
    T = len(sm)
    q_out = np.zeros((T, desc.num_q_heads, desc.head_dim), dtype=np.uint16)
    rc = lib().orc_rope_kv_write(C.byref(desc), _p(qkv), _p(pos), _p(cs), cs.shape[0], _p(q_out),
                                 _p(k_cache), _p(v_cache), _p(sm), T, _p(ks), _p(vs))
    if rc:
        raise ValueError("slot out of range")
    return q_out


def o_proj(a, w, bias=None, residual=None):
    """Output projection; a [T,K], w [N,K], bias [N], residual [T,N] as bf16 bits (uint16).
    Returns (out bf16 bits [T,N], exact float64 [T,N])."""
    a, w = _c(a, np.uint16), _c(w, np.uint16)
    b, r = _c(bias, np.uint16), _c(residual, np.uint16)
    T, K = a.shape
    N = w.shape[0]
    assert w.shape[1] == K
    out = np.zeros((T, N), dtype=np.uint16)
    exact = np.zeros((T, N), dtype=np.float64)
    lib().orc_o_proj(_p(a), _p(w), _p(b), _p(r), _p(out), _p(exact), T, N, K)
    return out, exact


def attn_f64(desc, q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q=None, sinks=None,
             k_scale=None, v_scale=None):
    """Definitional fp64 attention; returns (out [T,Hq,D] float64, lse [T,Hq] float64)."""
    T = desc.num_q_tokens
    out = np.zeros((T, desc.num_q_heads, desc.head_dim), dtype=np.float64)
    lse = np.zeros((T, desc.num_q_heads), dtype=np.float64)
    a, keep = _host_args(q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q, sinks,
                         k_scale, v_scale)
    rc = lib().orc_attn_f64(C.byref(desc), C.byref(a), _p(out), _p(lse))
    if rc:
        raise ValueError("malformed batch (query before position 0)")
    return out, lse


def splitkv_f64(desc, P, nparts, q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q=None,
                k_scale=None, v_scale=None):
    T = desc.num_q_tokens
    ml = np.zeros((T, desc.num_q_heads, nparts, 2), dtype=np.float64)
    acc = np.zeros((T, desc.num_q_heads, nparts, desc.head_dim), dtype=np.float64)
    a, keep = _host_args(q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q, None, k_scale,
                         v_scale)
    lib().orc_splitkv_partials_f64(C.byref(desc), C.byref(a), P, nparts, _p(ml), _p(acc))
    return ml, acc


def lse_merge_f64(ml, acc, sinks=None):
    T, Hq, nparts, D = acc.shape
    out = np.zeros((T, Hq, D), dtype=np.float64)
    lse = np.zeros((T, Hq), dtype=np.float64)
    s = _c(sinks, np.float32)
    lib().orc_lse_merge_f64(T, Hq, nparts, D, _p(np.ascontiguousarray(ml)),
                            _p(np.ascontiguousarray(acc)), _p(s), _p(out), _p(lse))
    return out, lse


def attn_bf16(desc, q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q=None, sinks=None,
              k_scale=None, v_scale=None, num_threads=0):
    """CPU baseline path (fp32 accumulate, OpenMP); returns bf16 bits [T,Hq,D] as uint16."""
    T = desc.num_q_tokens
    out = np.zeros((T, desc.num_q_heads, desc.head_dim), dtype=np.uint16)
    lse = np.zeros((T, desc.num_q_heads), dtype=np.float32)
    a, keep = _host_args(q, k_cache, v_cache, block_table, seq_lens, cu_seqlens_q, sinks,
                         k_scale, v_scale, out=out, lse=lse)
    rc = lib().orc_attn_bf16(C.byref(desc), C.byref(a), num_threads)
    if rc:
        raise ValueError(f"orc_attn_bf16 failed: {rc}")
    return out, lse


def fp8_encode(x):
    f = lib().orc_fp8_e4m3_encode
    return np.array([f(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()],
                    dtype=np.uint8).reshape(np.shape(x))


def fp8_decode(b):
    f = lib().orc_fp8_e4m3_decode
    return np.array([f(int(v)) for v in np.asarray(b, dtype=np.uint8).ravel()],
                    dtype=np.float32).reshape(np.shape(b))
