//! Raw declarations of `include/eidola_attn.h` and `include/eidola_sched.h`, field for field
//! and argument for argument.  Everything here is `unsafe` to call: pointers marked "device"
//! in the headers are HIP device pointers, `hip_stream` is a `hipStream_t`.  The safe layer is
//! the `eidola-attn` crate.
#![no_std]
#![allow(non_camel_case_types)]

use core::ffi::{c_char, c_void};

pub const EID_VERSION_MAJOR: u32 = 0;
pub const EID_VERSION_MINOR: u32 = 1;

pub const EID_OK: i32 = 0;
pub const EID_ERR_INVALID_ARG: i32 = -1;
pub const EID_ERR_UNSUPPORTED: i32 = -2;
pub const EID_ERR_WORKSPACE: i32 = -3;
pub const EID_ERR_HIP: i32 = -4;
pub const EID_ERR_NO_BLOCKS: i32 = -5;

pub const EID_KV_BF16: i32 = 0;
pub const EID_KV_FP8_E4M3: i32 = 1;

/// Size of the library's own split-KV workspace (`eid_attn_decode_noalloc`).
pub const EID_STATIC_WORKSPACE_BYTES: usize = 32 << 20;

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct eid_attn_desc {
    pub struct_size: u32,
    pub num_seqs: i32,
    pub num_q_tokens: i32,
    pub max_q_len: i32,
    pub max_kv_len: i32,
    pub num_q_heads: i32,
    pub num_kv_heads: i32,
    pub head_dim: i32,
    pub block_size: i32,
    pub max_blocks_per_seq: i32,
    pub num_blocks: i64,
    pub softmax_scale: f32,
    pub window: i32,
    pub kv_dtype: i32,
    pub partition_size: i32,
    pub sum_kv_len: i64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct eid_attn_args {
    pub q: *const c_void,
    pub out: *mut c_void,
    pub lse: *mut f32,
    pub k_cache: *const c_void,
    pub v_cache: *const c_void,
    pub block_table: *const i32,
    pub cu_seqlens_q: *const i32,
    pub seq_lens: *const i32,
    pub sinks: *const f32,
    pub k_scale: *const f32,
    pub v_scale: *const f32,
    pub workspace: *mut c_void,
    pub workspace_bytes: usize,
    pub split_done_event: *mut c_void,
    pub k_new: *const c_void,
    pub v_new: *const c_void,
    pub seq_lens_host: *const i32,
    pub cu_seqlens_q_host: *const i32,
    pub block_table_host: *const i32,
}

/// Opaque scheduler handle (`eid_sched_create` / `eid_sched_destroy`).
#[repr(C)]
pub struct eid_sched {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct eid_sched_config {
    pub struct_size: u32,
    pub block_size: i32,
    pub num_blocks: i64,
    pub max_blocks_per_seq: i32,
    pub prefix_reuse: i32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct eid_batch_info {
    pub num_seqs: i32,
    pub num_q_tokens: i32,
    pub max_q_len: i32,
    pub max_kv_len: i32,
    pub sum_kv_len: i64,
}

unsafe extern "C" {
    pub fn eid_kv_write(
        desc: *const eid_attn_desc,
        k_new: *const c_void,
        v_new: *const c_void,
        k_cache: *mut c_void,
        v_cache: *mut c_void,
        slot_mapping: *const i64,
        num_tokens: i32,
        k_scale: *const f32,
        v_scale: *const f32,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_rope_kv_write(
        desc: *const eid_attn_desc,
        qkv: *const c_void,
        positions: *const i32,
        cos_sin: *const f32,
        max_pos: i32,
        q_out: *mut c_void,
        k_cache: *mut c_void,
        v_cache: *mut c_void,
        slot_mapping: *const i64,
        num_tokens: i32,
        k_scale: *const f32,
        v_scale: *const f32,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_attn_decode(
        desc: *const eid_attn_desc,
        args: *const eid_attn_args,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_attn_decode_noalloc(
        desc: *const eid_attn_desc,
        args: *const eid_attn_args,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_attn_varlen(
        desc: *const eid_attn_desc,
        args: *const eid_attn_args,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_lse_merge(
        desc: *const eid_attn_desc,
        args: *const eid_attn_args,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_o_proj(
        attn_out: *const c_void,
        weight: *const c_void,
        bias: *const c_void,
        residual: *const c_void,
        out: *mut c_void,
        num_tokens: i32,
        out_features: i32,
        in_features: i32,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_qkv_rope_kv_write(
        desc: *const eid_attn_desc,
        hidden: *const c_void,
        weight: *const c_void,
        bias: *const c_void,
        in_features: i32,
        positions: *const i32,
        cos_sin: *const f32,
        max_pos: i32,
        q_out: *mut c_void,
        k_cache: *mut c_void,
        v_cache: *mut c_void,
        slot_mapping: *const i64,
        num_tokens: i32,
        k_scale: *const f32,
        v_scale: *const f32,
        hip_stream: *mut c_void,
    ) -> i32;

    pub fn eid_workspace_bytes(desc: *const eid_attn_desc) -> usize;

    pub fn eid_partition_size(desc: *const eid_attn_desc) -> i32;

    pub fn eid_last_error() -> *const c_char;

    pub fn eid_version() -> u32;

    pub fn eid_sched_create(cfg: *const eid_sched_config, out: *mut *mut eid_sched) -> i32;

    pub fn eid_sched_destroy(s: *mut eid_sched);

    pub fn eid_sched_add_seq(
        s: *mut eid_sched,
        seq_id: i64,
        prompt: *const i32,
        n: i32,
        cached_tokens: *mut i32,
    ) -> i32;

    pub fn eid_sched_free_seq(s: *mut eid_sched, seq_id: i64) -> i32;

    pub fn eid_sched_seq_len(s: *const eid_sched, seq_id: i64) -> i32;

    pub fn eid_sched_free_blocks(s: *const eid_sched) -> i64;

    pub fn eid_sched_block_refs(s: *const eid_sched, block: i64) -> i32;

    pub fn eid_sched_build_batch(
        s: *mut eid_sched,
        seq_ids: *const i64,
        q_lens: *const i32,
        num_seqs: i32,
        new_tokens: *const i32,
        block_table: *mut i32,
        slot_mapping: *mut i64,
        cu_seqlens_q: *mut i32,
        seq_lens: *mut i32,
        positions: *mut i32,
        info: *mut eid_batch_info,
    ) -> i32;
}
