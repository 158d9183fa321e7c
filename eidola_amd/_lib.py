"""ctypes binding of libeidola_attn_hip.so (the C ABI declared in include/eidola_attn.h).

The reference (eidola-ai/eidola) has no operator or FFI interface for this path — its only
engine seam is OpenAI-compatible HTTP (crates/eidola-server/src/backend.rs:87-108) — so the
structures below mirror this repository's own header field for field.
"""
import ctypes as C
import os

KV_BF16 = 0
KV_FP8_E4M3 = 1

EID_OK = 0
EID_ERR_INVALID_ARG = -1
EID_ERR_UNSUPPORTED = -2
EID_ERR_WORKSPACE = -3
EID_ERR_HIP = -4
EID_ERR_NO_BLOCKS = -5
STATIC_WORKSPACE_BYTES = 32 << 20   # EID_STATIC_WORKSPACE_BYTES of the header

_STATUS_NAMES = {
    EID_ERR_INVALID_ARG: "EID_ERR_INVALID_ARG",
    EID_ERR_UNSUPPORTED: "EID_ERR_UNSUPPORTED",
    EID_ERR_WORKSPACE: "EID_ERR_WORKSPACE",
    EID_ERR_HIP: "EID_ERR_HIP",
    EID_ERR_NO_BLOCKS: "EID_ERR_NO_BLOCKS",
}


class EidError(RuntimeError):
    """A non-zero eid_status, carrying the code and the library's thread-local message."""

    def __init__(self, status, message):
        self.status = status
        self.name = _STATUS_NAMES.get(status, str(status))
        super().__init__(f"{self.name}: {message}")


class AttnDesc(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("num_seqs", C.c_int32),
        ("num_q_tokens", C.c_int32),
        ("max_q_len", C.c_int32),
        ("max_kv_len", C.c_int32),
        ("num_q_heads", C.c_int32),
        ("num_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("block_size", C.c_int32),
        ("max_blocks_per_seq", C.c_int32),
        ("num_blocks", C.c_int64),
        ("softmax_scale", C.c_float),
        ("window", C.c_int32),
        ("kv_dtype", C.c_int32),
        ("partition_size", C.c_int32),
        ("sum_kv_len", C.c_int64),
    ]


class AttnArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p),
        ("out", C.c_void_p),
        ("lse", C.c_void_p),
        ("k_cache", C.c_void_p),
        ("v_cache", C.c_void_p),
        ("block_table", C.c_void_p),
        ("cu_seqlens_q", C.c_void_p),
        ("seq_lens", C.c_void_p),
        ("sinks", C.c_void_p),
        ("k_scale", C.c_void_p),
        ("v_scale", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("split_done_event", C.c_void_p),
        ("k_new", C.c_void_p),
        ("v_new", C.c_void_p),
        ("seq_lens_host", C.c_void_p),
        ("cu_seqlens_q_host", C.c_void_p),
        ("block_table_host", C.c_void_p),
    ]


class SchedConfig(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("block_size", C.c_int32),
        ("num_blocks", C.c_int64),
        ("max_blocks_per_seq", C.c_int32),
        ("prefix_reuse", C.c_int32),
    ]


class BatchInfo(C.Structure):
    _fields_ = [
        ("num_seqs", C.c_int32),
        ("num_q_tokens", C.c_int32),
        ("max_q_len", C.c_int32),
        ("max_kv_len", C.c_int32),
        ("sum_kv_len", C.c_int64),
    ]


EXPORTS = ("eid_kv_write", "eid_rope_kv_write", "eid_qkv_rope_kv_write", "eid_attn_decode",
           "eid_attn_decode_noalloc", "eid_attn_varlen", "eid_lse_merge", "eid_o_proj",
           "eid_workspace_bytes", "eid_partition_size", "eid_last_error", "eid_version")
# only in the measurement build (include/eidola_attn_measure.h)
MEASURE_EXPORTS = ("eid_debug_set_timeline", "eid_debug_set_kernel_events",
                   "eid_debug_set_store_every_partition")
SCHED_EXPORTS = ("eid_sched_create", "eid_sched_destroy", "eid_sched_add_seq",
                 "eid_sched_free_seq", "eid_sched_seq_len", "eid_sched_free_blocks",
                 "eid_sched_block_refs", "eid_sched_build_batch")

_lib = None
_measure_lib = None


def lib_path():
    override = os.environ.get("EID_ATTN_LIB")   # an alternative build of the same ABI
    if override:
        return override
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc",
                        "libeidola_attn_hip.so")


def measure_lib_path():
    override = os.environ.get("EID_ATTN_MEASURE_LIB")
    if override:
        return override
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc",
                        "libeidola_attn_measure.so")


def load_measure_library():
    """The measurement build of the library (the same sources with -DEID_MEASURE): a second,
    independent copy in the process, with the two eid_debug_* hooks.  For benchmarks only."""
    global _measure_lib
    if _measure_lib is None:
        _measure_lib = _bind(measure_lib_path(), measure=True)
    return _measure_lib


def load_library():
    """Load the HIP library; raises (never falls back) when it has not been built."""
    global _lib
    if _lib is None:
        _lib = _bind(lib_path(), measure=False)
    return _lib


def _bind(path, measure):
    if not os.path.exists(path):
        raise EidError(EID_ERR_HIP, f"{path} is missing: run `python -c 'import "
                       "__graft_entry__ as g; g.build()'` or `make -C eidola_amd/csrc`")
    lib = C.CDLL(path)
    P = C.c_void_p
    lib.eid_kv_write.argtypes = [C.POINTER(AttnDesc), P, P, P, P, P, C.c_int32, P, P, P]
    lib.eid_kv_write.restype = C.c_int32
    lib.eid_rope_kv_write.argtypes = [C.POINTER(AttnDesc), P, P, P, C.c_int32, P, P, P, P,
                                      C.c_int32, P, P, P]
    lib.eid_rope_kv_write.restype = C.c_int32
    lib.eid_qkv_rope_kv_write.argtypes = [C.POINTER(AttnDesc), P, P, P, C.c_int32, P, P, C.c_int32,
                                          P, P, P, P, C.c_int32, P, P, P]
    lib.eid_qkv_rope_kv_write.restype = C.c_int32
    lib.eid_o_proj.argtypes = [P, P, P, P, P, C.c_int32, C.c_int32, C.c_int32, P]
    lib.eid_o_proj.restype = C.c_int32
    for name in ("eid_attn_decode", "eid_attn_decode_noalloc", "eid_attn_varlen", "eid_lse_merge"):
        fn = getattr(lib, name)
        fn.argtypes = [C.POINTER(AttnDesc), C.POINTER(AttnArgs), P]
        fn.restype = C.c_int32
    lib.eid_workspace_bytes.argtypes = [C.POINTER(AttnDesc)]
    lib.eid_workspace_bytes.restype = C.c_size_t
    lib.eid_partition_size.argtypes = [C.POINTER(AttnDesc)]
    lib.eid_partition_size.restype = C.c_int32
    lib.eid_last_error.argtypes = []
    lib.eid_last_error.restype = C.c_char_p
    lib.eid_version.argtypes = []
    lib.eid_version.restype = C.c_uint32
    if measure:
        lib.eid_debug_set_timeline.argtypes = [P, C.c_int64]
        lib.eid_debug_set_timeline.restype = None
        lib.eid_debug_set_kernel_events.argtypes = [P, P]
        lib.eid_debug_set_kernel_events.restype = None
        lib.eid_debug_set_store_every_partition.argtypes = [C.c_int32]
        lib.eid_debug_set_store_every_partition.restype = None
    # host-side scheduler (include/eidola_sched.h)
    lib.eid_sched_create.argtypes = [C.POINTER(SchedConfig), C.POINTER(P)]
    lib.eid_sched_create.restype = C.c_int32
    lib.eid_sched_destroy.argtypes = [P]
    lib.eid_sched_destroy.restype = None
    lib.eid_sched_add_seq.argtypes = [P, C.c_int64, P, C.c_int32, C.POINTER(C.c_int32)]
    lib.eid_sched_add_seq.restype = C.c_int32
    lib.eid_sched_free_seq.argtypes = [P, C.c_int64]
    lib.eid_sched_free_seq.restype = C.c_int32
    lib.eid_sched_seq_len.argtypes = [P, C.c_int64]
    lib.eid_sched_seq_len.restype = C.c_int32
    lib.eid_sched_free_blocks.argtypes = [P]
    lib.eid_sched_free_blocks.restype = C.c_int64
    lib.eid_sched_block_refs.argtypes = [P, C.c_int64]
    lib.eid_sched_block_refs.restype = C.c_int32
    lib.eid_sched_build_batch.argtypes = [P, P, P, C.c_int32, P, P, P, P, P, P,
                                          C.POINTER(BatchInfo)]
    lib.eid_sched_build_batch.restype = C.c_int32
    return lib


def check(status):
    if status != EID_OK:
        raise EidError(status, load_library().eid_last_error().decode())


def version():
    v = load_library().eid_version()
    return v >> 16, v & 0xFFFF
