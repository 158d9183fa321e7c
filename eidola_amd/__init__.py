"""eidola_amd — MI355X (gfx950) ragged-batch paged sink-attention path.

Host-side mirror of the C ABI in ``include/eidola_attn.h``.  The compute lives in
``eidola_amd/csrc`` (hand-written HIP); torch is used only to own device memory and
streams.  There is no CPU fallback: every operator raises if the HIP library is missing.
"""
from ._lib import (EidError, AttnDesc, AttnArgs, KV_BF16, KV_FP8_E4M3, STATIC_WORKSPACE_BYTES,
                   lib_path, load_library, version)
from .sched import Scheduler, BuiltBatch
from .ops import (AttnGeometry, kv_write, rope_kv_write, qkv_rope_kv_write, yarn_cos_sin, o_proj, attn_decode, attn_decode_noalloc, attn_varlen,
                  lse_merge, workspace_bytes, partition_size, make_desc, prepare, PreparedCall)

__all__ = [
    "EidError", "AttnDesc", "AttnArgs", "KV_BF16", "KV_FP8_E4M3", "STATIC_WORKSPACE_BYTES", "lib_path", "load_library",
    "version", "AttnGeometry", "kv_write", "rope_kv_write", "qkv_rope_kv_write", "yarn_cos_sin", "o_proj", "attn_decode", "attn_decode_noalloc", "attn_varlen",
    "lse_merge", "workspace_bytes", "partition_size", "make_desc", "prepare", "PreparedCall",
    "Scheduler", "BuiltBatch",
]
