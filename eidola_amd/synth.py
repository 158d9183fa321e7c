"""Seeded synthetic ragged batches: the five benchmark configurations and scaled-down twins.

Metadata (context lengths, query lengths, block tables, slot mappings) always comes from a
counter-based SplitMix64 stream in numpy, so it is identical on every host.  Tensor
contents come from the same stream for small cases (`normal_bf16`); multi-gigabyte KV pools
are filled on the GPU with a seeded torch generator instead (`fill_pool_gpu`).
"""
import math
from dataclasses import dataclass, field, replace

import numpy as np

from ._lib import KV_BF16, KV_FP8_E4M3
from .ops import AttnGeometry

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)

# tensor ids of the counter-based stream
TID_Q, TID_K, TID_V, TID_SINK, TID_LEN, TID_PERM, TID_PRIOR = 1, 2, 3, 4, 5, 6, 7


def mix64(seed, tensor_id, index):
    """SplitMix64 finaliser of (seed, tensor_id, index); index may be an array."""
    with np.errstate(over="ignore"):
        z = (np.asarray(index, dtype=np.uint64)
             + np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15)
             + np.uint64(tensor_id) * np.uint64(0xD1B54A32D192ED03)
             + np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform(seed, tensor_id, index):
    """Uniform in (0, 1) with 53 random bits."""
    return ((mix64(seed, tensor_id, index) >> np.uint64(11)).astype(np.float64) + 0.5) / float(1 << 53)


def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (uint16)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    r = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def normal_bf16(shape, seed, tensor_id, first_index=0):
    """i.i.d. N(0,1) by Box-Muller on two uniforms keyed by element index, rounded to bf16."""
    n = int(np.prod(shape))
    idx = np.arange(first_index, first_index + n, dtype=np.uint64)
    u1 = uniform(seed, tensor_id, idx * np.uint64(2))
    u2 = uniform(seed, tensor_id, idx * np.uint64(2) + np.uint64(1))
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * math.pi * u2)
    return f32_to_bf16_bits(z.astype(np.float32)).reshape(shape)


def randint(n, lo, hi, seed, tensor_id):
    """n integers uniform in [lo, hi]."""
    u = uniform(seed, tensor_id, np.arange(n, dtype=np.uint64))
    return (lo + np.floor(u * (hi - lo + 1))).astype(np.int64).clip(lo, hi)


def permutation(n, seed, tensor_id):
    """A permutation of 0..n-1: stable argsort of n keyed 64-bit draws."""
    return np.argsort(mix64(seed, tensor_id, np.arange(n, dtype=np.uint64)), kind="stable").astype(np.int32)


@dataclass
class Batch:
    name: str
    geom: AttnGeometry
    seq_lens: np.ndarray        # int32 [S], KV length after this step's append
    q_lens: np.ndarray          # int32 [S]
    block_table: np.ndarray     # int32 [S, max_blocks_per_seq]
    num_blocks: int
    seed: int
    cu_seqlens_q: np.ndarray = field(init=False)
    slot_mapping: np.ndarray = field(init=False)  # int64 [T], slots of this step's new tokens

    def __post_init__(self):
        self.seq_lens = self.seq_lens.astype(np.int32)
        self.q_lens = self.q_lens.astype(np.int32)
        self.cu_seqlens_q = np.concatenate([[0], np.cumsum(self.q_lens)]).astype(np.int32)
        slots = []
        B = self.geom.block_size
        for s in range(self.num_seqs):
            pos = np.arange(self.seq_lens[s] - self.q_lens[s], self.seq_lens[s])
            slots.append(self.block_table[s, pos // B].astype(np.int64) * B + pos % B)
        self.slot_mapping = np.concatenate(slots).astype(np.int64)

    @property
    def num_seqs(self):
        return len(self.seq_lens)

    @property
    def num_q_tokens(self):
        return int(self.q_lens.sum())

    @property
    def max_q_len(self):
        return int(self.q_lens.max())

    @property
    def max_kv_len(self):
        return int(self.seq_lens.max())

    def all_slots(self, s):
        """Slots of every context position of sequence s."""
        B = self.geom.block_size
        pos = np.arange(self.seq_lens[s])
        return self.block_table[s, pos // B].astype(np.int64) * B + pos % B

    def with_geom(self, **kw):
        b = replace(self, geom=replace(self.geom, **kw))
        return b


def build_block_table(seq_lens, num_blocks, seed, block_size=16, max_blocks_per_seq=None,
                      perm_offset=0, shuffle=True):
    """Physical pages = consecutive slices of a seeded permutation of the pool
    (shuffle=False: of 0..num_blocks-1 in order, for locality experiments)."""
    nblk = (np.asarray(seq_lens, dtype=np.int64) + block_size - 1) // block_size
    total = int(nblk.sum())
    if perm_offset + total > num_blocks:
        raise ValueError(f"pool of {num_blocks} blocks cannot hold {perm_offset + total}")
    perm = permutation(num_blocks, seed, TID_PERM) if shuffle else np.arange(num_blocks, dtype=np.int32)
    mb = int(max_blocks_per_seq or nblk.max())
    if mb < nblk.max():
        raise ValueError("max_blocks_per_seq too small")
    bt = np.zeros((len(seq_lens), mb), dtype=np.int32)
    off = perm_offset
    for s, n in enumerate(nblk):
        bt[s, :n] = perm[off:off + n]
        off += int(n)
    return bt


def _geom(**kw):
    return AttnGeometry(num_q_heads=64, num_kv_heads=8, head_dim=64, block_size=16,
                        softmax_scale=0.125, **kw)


def config1():
    """Plumbing: 4 decodes with contexts {37,128,511,1000}, 128-block pool, seed 0."""
    L = np.array([37, 128, 511, 1000])
    bt = build_block_table(L, 128, 0)
    return Batch("config1_plumbing", _geom(), L, np.ones(4, dtype=np.int32), bt, 128, 0)


def config2(window=0, scale=1.0, num_blocks=300_000, perm_offset=0, shuffle=True):
    """Decode continuous batch: 64 sequences, contexts U{1..8192*scale}."""
    seed = 2
    hi = max(1, int(8192 * scale))
    L = randint(64, 1, hi, seed, TID_LEN)
    bt = build_block_table(L, num_blocks, seed, max_blocks_per_seq=max(1, (hi + 15) // 16),
                           perm_offset=perm_offset, shuffle=shuffle)
    name = f"config2_decode_{'w%d' % window if window else 'full'}"
    return Batch(name, _geom(window=window), L, np.ones(64, dtype=np.int32), bt, num_blocks, seed)


def config3(scale=1.0, num_blocks=300_000, chunk=512, perm_offset=0):
    """Mixed batch: 8 prefill chunks of `chunk` tokens at prior offsets U{0..4096*scale}
    plus 120 decodes with contexts U{1..8192*scale}."""
    seed = 3
    prior = randint(8, 0, int(4096 * scale), seed, TID_PRIOR)
    dec = randint(120, 1, max(1, int(8192 * scale)), seed, TID_LEN)
    L = np.concatenate([prior + chunk, dec])
    q = np.concatenate([np.full(8, chunk), np.ones(120)]).astype(np.int32)
    bt = build_block_table(L, num_blocks, seed, perm_offset=perm_offset)
    return Batch("config3_mixed_prefill_decode", _geom(), L, q, bt, num_blocks, seed)


def config4(scale=1.0, num_blocks=None, perm_offset=0):
    """fp8 KV decode: 256 sequences, contexts log-uniform in [128, 32768*scale]."""
    seed = 4
    hi = max(129.0, 32768 * scale)
    u = uniform(seed, TID_LEN, np.arange(256, dtype=np.uint64))
    L = np.rint(np.exp(math.log(128.0) + u * (math.log(hi) - math.log(128.0)))).astype(np.int64)
    need = int(((L + 15) // 16).sum())
    nb = num_blocks or max(120_000 if scale == 1.0 else 0, need + 64)
    bt = build_block_table(L, nb, seed, perm_offset=perm_offset)
    return Batch("config4_fp8_decode", _geom(kv_dtype=KV_FP8_E4M3), L, np.ones(256, dtype=np.int32),
                 bt, nb, seed)


def config5(layer=0, scale=1.0, num_blocks=None, partition=512, perm_offset=0):
    """Speculative verify: 128 sequences x 5 query rows, contexts U{1024*scale..65536*scale};
    layer 0 = full attention, layer 1 = 128-token window."""
    seed = 5
    lo, hi = max(8, int(1024 * scale)), max(16, int(65536 * scale))
    L = randint(128, lo, hi, seed, TID_LEN)
    need = int(((L + 15) // 16).sum())
    nb = num_blocks or max(300_000 if scale == 1.0 else 0, need + 64)
    bt = build_block_table(L, nb, seed + 100 * layer, perm_offset=perm_offset)
    window = 128 if layer % 2 == 1 else 0
    return Batch(f"config5_verify_layer{layer}", _geom(window=window, partition_size=partition),
                 L, np.full(128, 5, dtype=np.int32), bt, nb, seed)


# ---------------------------------------------------------------------------------------
# algorithmic work of a batch: the bytes and flops the roofline fractions are quoted on
# ---------------------------------------------------------------------------------------
def algorithmic_work(batch, rows="all", include_kv_write=False):
    """bytes = sum_seq L_eff * 2*Hkv*D*sizeof(kv) + Q rows + O rows + touched block-table
    entries * 4 + sinks; flops = 4*D*Hq * (unmasked query-key pairs).
    rows: "all", "short" (q_len <= 6) or "long" (q_len > 6) selects the sequences counted."""
    g = batch.geom
    kvsz = 1 if g.kv_dtype == KV_FP8_E4M3 else 2
    per_tok = 2 * g.num_kv_heads * g.head_dim * kvsz
    row_bytes = g.num_q_heads * g.head_dim * 2
    W = g.window
    nbytes, pairs, qtok, ctx = g.num_q_heads * 4, 0, 0, 0
    for L, q in zip(batch.seq_lens.tolist(), batch.q_lens.tolist()):
        if rows == "short" and q > 6:
            continue
        if rows == "long" and q <= 6:
            continue
        p0 = L - q
        lo = max(0, p0 - W + 1) if W > 0 else 0
        l_eff = L - lo
        nbytes += l_eff * per_tok + 2 * q * row_bytes + ((L - 1) // 16 - lo // 16 + 1) * 4
        for i in range(q):
            p = p0 + i
            pairs += min(W, p + 1) if W > 0 else p + 1
        qtok += q
        ctx += l_eff
        if include_kv_write:
            nbytes += q * g.num_kv_heads * g.head_dim * 2 * (2 + kvsz)
    return {"bytes": int(nbytes), "flops": int(4 * g.head_dim * g.num_q_heads * pairs),
            "q_tokens": int(qtok), "ctx_tokens": int(ctx), "pairs": int(pairs)}


# ---------------------------------------------------------------------------------------
# GPU-side pool fill for the large configurations (torch used as a device RNG only)
# ---------------------------------------------------------------------------------------
def fill_pool_gpu(geom, k_cache, v_cache, seed, chunk_slots=1 << 16):
    """Fill every slot of a paged pool with N(0,1) values.  bf16 pools take the values as
    they are; fp8 pools are written through the library's own kv_write with
    scale[h] = absmax_h / 448 over the whole generated source.  Returns (k_scale, v_scale)
    (None for bf16)."""
    import torch
    from . import ops
    dev = k_cache.device
    nslots = k_cache.shape[0] * k_cache.shape[1]
    H, D = geom.num_kv_heads, geom.head_dim

    def chunks():
        for ci, a in enumerate(range(0, nslots, chunk_slots)):
            b = min(nslots, a + chunk_slots)
            gen = torch.Generator(device=dev)
            gen.manual_seed(seed * 1_000_003 + ci)
            kv = torch.randn((2, b - a, H, D), generator=gen, device=dev,
                             dtype=torch.float32).to(torch.bfloat16)
            yield a, b, kv

    if geom.kv_dtype == KV_BF16:
        kf = k_cache.view(nslots, H, D)
        vf = v_cache.view(nslots, H, D)
        for a, b, kv in chunks():
            kf[a:b] = kv[0]
            vf[a:b] = kv[1]
        return None, None
    amax = torch.zeros((2, H), dtype=torch.float32, device=dev)
    for a, b, kv in chunks():
        amax = torch.maximum(amax, kv.float().abs().amax(dim=(1, 3)))
    scales = (amax / 448.0).contiguous()
    k_scale, v_scale = scales[0].contiguous(), scales[1].contiguous()
    for a, b, kv in chunks():
        slots = torch.arange(a, b, dtype=torch.int64, device=dev)
        ops.kv_write(geom, kv[0].contiguous(), kv[1].contiguous(), k_cache, v_cache, slots,
                     k_scale, v_scale)
    return k_scale, v_scale
