"""Independent numpy restatement of paged sink-attention (TEST INFRASTRUCTURE ONLY).

Written separately from eid_oracle.c, with a different structure (gather the whole context
of a sequence first, then dense masked softmax), so that an indexing or masking mistake in
one of the two shows up as a disagreement.  No reference file exists to follow: the
definition is  out = sum_j e^(s_j-m) v_j / (e^(sink-m) + sum_j e^(s_j-m)),
s_j = scale * <q, k_j>, over keys max(0, p-W+1) <= j <= p.
"""
import numpy as np


def bf16_to_f64(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32).astype(np.float64)


def fp8_e4m3_to_f64(b):
    """Table-driven OCP e4m3fn decode (256 entries built from the format definition)."""
    tab = np.empty(256, dtype=np.float64)
    for code in range(256):
        s, e, m = code >> 7, (code >> 3) & 15, code & 7
        if e == 15 and m == 7:
            v = np.nan
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (8 + m) * 2.0 ** (e - 10)
        tab[code] = -v if s else v
    return tab[np.asarray(b, dtype=np.uint8)]


def fp8_e4m3_encode_np(x):
    """Nearest-even e4m3fn code by exhaustive search over the 254 finite codes, with
    saturation to +-448 and NaN -> 0x7F.  O(256) per value: for cross-checks only."""
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    vals = fp8_e4m3_to_f64(codes)
    x = np.asarray(x, dtype=np.float64)
    out = np.empty(x.shape, dtype=np.uint8)
    flat = x.ravel()
    o = out.ravel()
    for i, v in enumerate(flat):
        if np.isnan(v):
            o[i] = 0x7F
            continue
        v = min(max(v, -448.0), 448.0)
        d = np.abs(vals - v)
        best = np.flatnonzero(d == d.min())
        if len(best) > 1:   # tie: even mantissa; +-0 tie resolved by sign of v
            cand = [c for c in codes[best] if (c & 1) == 0]
            if len(cand) > 1:
                cand = [c for c in cand if bool(c & 0x80) == bool(np.signbit(v))]
            o[i] = cand[0]
        else:
            c = codes[best[0]]
            if vals[best[0]] == 0.0:
                c = 0x80 if np.signbit(v) else 0x00
            o[i] = c
    return out


def attention(q_bits, k_cache, v_cache, block_table, seq_lens, q_lens, *, num_kv_heads, scale,
              window=0, sinks=None, fp8=False, k_scale=None, v_scale=None, block_size=16):
    """q_bits [T,Hq,D] uint16; caches [NB,B,Hkv,D] uint16 (bf16 bits) or uint8 (fp8).
    Returns out [T,Hq,D] float64 and lse [T,Hq]."""
    q = bf16_to_f64(q_bits)
    T, Hq, D = q.shape
    G = Hq // num_kv_heads
    dec = fp8_e4m3_to_f64 if fp8 else bf16_to_f64
    out = np.zeros((T, Hq, D))
    lse = np.zeros((T, Hq))
    row = 0
    for s, (L, ql) in enumerate(zip(seq_lens, q_lens)):
        L, ql = int(L), int(ql)
        nblk = (L + block_size - 1) // block_size
        pages = block_table[s, :nblk]
        K = dec(k_cache[pages]).reshape(nblk * block_size, num_kv_heads, D)[:L]
        V = dec(v_cache[pages]).reshape(nblk * block_size, num_kv_heads, D)[:L]
        if fp8:
            K = K * np.asarray(k_scale, dtype=np.float64)[None, :, None]
            V = V * np.asarray(v_scale, dtype=np.float64)[None, :, None]
        pos = np.arange(L - ql, L)
        j = np.arange(L)
        allowed = j[None, :] <= pos[:, None]
        if window > 0:
            allowed &= (pos[:, None] - j[None, :]) < window
        for h in range(Hq):
            sc = scale * q[row:row + ql, h] @ K[:, h // G].T          # [ql, L]
            sc = np.where(allowed, sc, -np.inf)
            sink = -np.inf if sinks is None else float(sinks[h])
            m = np.maximum(sc.max(axis=1), sink)
            w = np.exp(sc - m[:, None])
            den = w.sum(axis=1) + np.exp(sink - m)
            out[row:row + ql, h] = (w @ V[:, h // G]) / den[:, None]
            lse[row:row + ql, h] = m + np.log(den)
        row += ql
    return out, lse
