"""Host-only checks of the C ABI: the library loads without a GPU, exports every symbol the
header declares, and rejects bad arguments before touching HIP."""
import ctypes as C
import os
import re

import pytest

import eidola_amd as ea
from eidola_amd import _lib
from eidola_amd._lib import AttnArgs, AttnDesc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def good_desc(**kw):
    d = ea.make_desc(ea.AttnGeometry(), num_seqs=4, num_q_tokens=4, max_q_len=1, max_kv_len=1000,
                     max_blocks_per_seq=63, num_blocks=128)
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "eidola_attn.h")).read()
    declared = set(re.findall(r"\b(eid_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    lib = ea.load_library()
    for name in declared:
        assert hasattr(lib, name), name
    assert ea.version() == (0, 1)


def test_struct_layout_matches_header():
    assert C.sizeof(AttnDesc) == 72
    assert AttnDesc.num_blocks.offset == 40 and AttnDesc.softmax_scale.offset == 48
    assert C.sizeof(AttnArgs) == 19 * 8


def test_workspace_and_partition_planning():
    d = good_desc()
    P = ea.partition_size(d)
    assert P % 64 == 0 and 64 <= P <= 4096
    # plan header, one int32 per sequence (pieces of an even split), then (m, l) and the outputs;
    # a run-time partition plans one more piece than whole partitions of 256 keys
    Pl, nparts, ws_rows, ml_off, acc_off = ea.ops.workspace_layout(d)
    assert Pl == P and ws_rows == 1 and nparts == (1000 + P - 1) // P + (1 if d.partition_size == 0 and P == 256 else 0)
    cells = 4 * 1 * 64 * nparts
    assert ml_off == 256 + 256 and acc_off == ml_off + (cells * 8 + 255) // 256 * 256
    assert ea.workspace_bytes(d) == acc_off + cells * 128
    d5 = ea.make_desc(ea.AttnGeometry(partition_size=512), num_seqs=128, num_q_tokens=640,
                      max_q_len=5, max_kv_len=65536, max_blocks_per_seq=4096, num_blocks=300000)
    assert ea.partition_size(d5) == 512
    assert ea.workspace_bytes(d5) == 256 + 512 + 128 * 5 * 64 * 128 * (8 + 128)
    # at least one sequence per CU (256 without a device to ask) and no span beyond 2,048
    # tokens: every sequence is planned as one work item, and the workspace shrinks to it
    dm = ea.make_desc(ea.AttnGeometry(), num_seqs=300, num_q_tokens=300, max_q_len=1,
                      max_kv_len=1300, max_blocks_per_seq=82, num_blocks=300000)
    assert ea.partition_size(dm) == 1344
    assert ea.workspace_bytes(dm) == 256 + 300 * 64 * (8 + 128)
    dm.max_kv_len, dm.max_blocks_per_seq = 2049, 129
    assert ea.partition_size(dm) == 256
    dm.num_seqs = dm.num_q_tokens = 255
    dm.max_kv_len = 1300
    assert ea.partition_size(dm) == 256
    dw = ea.make_desc(ea.AttnGeometry(window=128), num_seqs=64, num_q_tokens=64, max_q_len=1,
                      max_kv_len=8192, max_blocks_per_seq=512, num_blocks=300000)
    assert ea.workspace_bytes(dw) < ea.workspace_bytes(good_desc(num_seqs=64, num_q_tokens=64,
                                                                 max_kv_len=8192,
                                                                 max_blocks_per_seq=512))


@pytest.mark.parametrize("field,value,status", [
    ("struct_size", 12, "EID_ERR_INVALID_ARG"),
    ("head_dim", 128, "EID_ERR_UNSUPPORTED"),
    ("block_size", 32, "EID_ERR_UNSUPPORTED"),
    ("num_q_heads", 32, "EID_ERR_UNSUPPORTED"),
    ("num_kv_heads", 0, "EID_ERR_INVALID_ARG"),
    ("kv_dtype", 7, "EID_ERR_INVALID_ARG"),
    ("num_seqs", 0, "EID_ERR_INVALID_ARG"),
    ("max_q_len", 0, "EID_ERR_INVALID_ARG"),
    ("max_kv_len", 5000, "EID_ERR_INVALID_ARG"),       # 63 blocks cannot hold it
    ("softmax_scale", 0.0, "EID_ERR_INVALID_ARG"),
    ("softmax_scale", float("nan"), "EID_ERR_INVALID_ARG"),
    ("window", -1, "EID_ERR_INVALID_ARG"),
    ("sum_kv_len", 999, "EID_ERR_INVALID_ARG"),          # below max_kv_len
    ("partition_size", 100, "EID_ERR_INVALID_ARG"),
    ("partition_size", 8192, "EID_ERR_INVALID_ARG"),
    ("num_blocks", 0, "EID_ERR_INVALID_ARG"),
])
def test_bad_descriptors_are_rejected_without_a_gpu(field, value, status):
    lib = ea.load_library()
    d = good_desc(**{field: value})
    assert ea.workspace_bytes(d) == 0
    rc = lib.eid_attn_decode(C.byref(d), C.byref(AttnArgs()), None)
    assert rc != 0
    with pytest.raises(ea.EidError) as e:
        _lib.check(rc)
    assert e.value.name == status and str(e.value)


def test_bad_arguments_are_rejected_without_a_gpu():
    lib = ea.load_library()
    d = good_desc()
    a = AttnArgs()
    assert lib.eid_attn_decode(C.byref(d), None, None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_attn_decode(None, C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_attn_decode(C.byref(d), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    assert b"non-NULL" in lib.eid_last_error()
    for f in ("q", "out", "k_cache", "v_cache", "block_table", "seq_lens"):
        setattr(a, f, 0x1000)
    a.k_cache = 0x1008                       # misaligned
    assert lib.eid_attn_decode(C.byref(d), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    assert b"aligned" in lib.eid_last_error()
    a.k_cache = 0x1000
    assert lib.eid_attn_decode(C.byref(d), C.byref(a), None) == _lib.EID_ERR_WORKSPACE
    a.workspace, a.workspace_bytes = 0x2000, 16
    assert lib.eid_attn_decode(C.byref(d), C.byref(a), None) == _lib.EID_ERR_WORKSPACE
    a.workspace, a.workspace_bytes = 0x2010, ea.workspace_bytes(d)
    assert lib.eid_attn_decode(C.byref(d), C.byref(a), None) == _lib.EID_ERR_WORKSPACE
    # varlen needs cu_seqlens_q; decode needs q_len == 1 everywhere
    a.workspace = 0x2000
    assert lib.eid_attn_varlen(C.byref(d), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    d2 = good_desc(num_q_tokens=20, max_q_len=5)
    a.workspace_bytes = ea.workspace_bytes(d2)
    assert lib.eid_attn_decode(C.byref(d2), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    # fp8 needs scales
    d8 = good_desc(kv_dtype=ea.KV_FP8_E4M3)
    a.workspace_bytes = ea.workspace_bytes(d8)
    assert lib.eid_attn_decode(C.byref(d8), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    assert b"scale" in lib.eid_last_error()


def test_noalloc_decode_validates_and_bounds_its_static_workspace_without_a_gpu():
    lib = ea.load_library()
    header = open(os.path.join(ROOT, "include", "eidola_attn.h")).read()
    m = re.search(r"#define EID_STATIC_WORKSPACE_BYTES \((\d+)u << (\d+)\)", header)
    assert int(m.group(1)) << int(m.group(2)) == ea.STATIC_WORKSPACE_BYTES
    a = AttnArgs()
    d = good_desc()
    assert lib.eid_attn_decode_noalloc(C.byref(d), None, None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_attn_decode_noalloc(C.byref(d), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG
    for f in ("q", "out", "k_cache", "v_cache", "block_table", "seq_lens"):
        setattr(a, f, 0x1000)
    # a batch whose partials cannot fit the static array is turned away before any launch
    big = ea.make_desc(ea.AttnGeometry(partition_size=128), num_seqs=512, num_q_tokens=512,
                       max_q_len=1, max_kv_len=8192, max_blocks_per_seq=512, num_blocks=300000)
    assert ea.workspace_bytes(big) > ea.STATIC_WORKSPACE_BYTES
    assert lib.eid_attn_decode_noalloc(C.byref(big), C.byref(a), None) == _lib.EID_ERR_WORKSPACE
    assert b"static" in lib.eid_last_error()
    d5 = good_desc(num_q_tokens=20, max_q_len=5)
    assert lib.eid_attn_decode_noalloc(C.byref(d5), C.byref(a), None) == _lib.EID_ERR_INVALID_ARG


def test_kv_write_validation_without_a_gpu():
    lib = ea.load_library()
    d = good_desc()
    assert lib.eid_kv_write(C.byref(d), None, None, None, None, None, 0, None, None, None) == 0
    assert lib.eid_kv_write(C.byref(d), None, None, None, None, None, 3, None, None,
                            None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_kv_write(C.byref(d), None, None, None, None, None, -1, None, None,
                            None) == _lib.EID_ERR_INVALID_ARG
    d8 = good_desc(kv_dtype=ea.KV_FP8_E4M3)
    assert lib.eid_kv_write(C.byref(d8), 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 3, None, None,
                            None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_last_error() != b""


def test_o_proj_validation_without_a_gpu():
    lib = ea.load_library()
    ok = 0x1000
    assert lib.eid_o_proj(None, None, None, None, None, 0, 2880, 4096, None) == 0
    assert lib.eid_o_proj(ok, ok, None, None, None, 4, 2880, 4096, None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_o_proj(ok, ok, None, None, ok, -1, 2880, 4096, None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_o_proj(ok, ok, None, None, ok, 4, 2880, 4100, None) == _lib.EID_ERR_UNSUPPORTED
    assert lib.eid_o_proj(ok, ok, None, None, ok, 4, 2888, 4096, None) == _lib.EID_ERR_UNSUPPORTED
    assert lib.eid_o_proj(ok, ok, ok + 8, None, ok + 0x100, 4, 2880, 4096, None) == _lib.EID_ERR_INVALID_ARG
    assert lib.eid_o_proj(ok, ok, None, None, ok, 4, 2880, 4096, None) == _lib.EID_ERR_INVALID_ARG  # out aliases attn_out
    assert b"alias" in lib.eid_last_error()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "lib_path", lambda: str(tmp_path / "nope.so"))
    with pytest.raises(ea.EidError):
        _lib.load_library()
