//! Safe layer over `eidola-attn-sys`.
//!
//! Host-side state (the block allocator and batch builder, descriptor validation, error
//! strings) is fully safe here.  Launch functions stay `unsafe fn`: they take HIP device
//! pointers and a `hipStream_t` that only the caller can vouch for, and the kernels run
//! asynchronously on that stream after the call has returned.
//!
//! Errors follow the workspace's convention: one `thiserror` enum whose variants are the
//! distinct failure modes, so a caller never parses strings.

use std::ffi::{c_void, CStr};
use std::ptr;

use eidola_attn_sys as sys;

/// Failure modes of the library, one per status code of `include/eidola_attn.h`.
#[derive(Debug, Clone, thiserror::Error)]
pub enum AttnError {
    /// Null pointer, bad shape, misalignment, wrong `struct_size`.
    #[error("invalid argument: {message}")]
    InvalidArg { message: String },
    /// Geometry or dtype outside what this version of the library builds.
    #[error("unsupported geometry: {message}")]
    Unsupported { message: String },
    /// Workspace missing, misaligned or smaller than `workspace_bytes()` asks for.
    #[error("workspace too small or misaligned: {message}")]
    Workspace { message: String },
    /// A HIP runtime call or kernel launch failed.
    #[error("HIP failure: {message}")]
    Hip { message: String },
    /// The KV pool cannot hold the request; no sequence was changed.
    #[error("KV pool exhausted: {message}")]
    NoBlocks { message: String },
    /// A status code this wrapper does not know (a newer library).
    #[error("status {code}: {message}")]
    Other { code: i32, message: String },
}

fn last_error() -> String {
    // SAFETY: eid_last_error returns a NUL-terminated thread-local string owned by the library.
    unsafe { CStr::from_ptr(sys::eid_last_error()) }.to_string_lossy().into_owned()
}

fn check(rc: i32) -> Result<(), AttnError> {
    if rc == sys::EID_OK {
        return Ok(());
    }
    let message = last_error();
    Err(match rc {
        sys::EID_ERR_INVALID_ARG => AttnError::InvalidArg { message },
        sys::EID_ERR_UNSUPPORTED => AttnError::Unsupported { message },
        sys::EID_ERR_WORKSPACE => AttnError::Workspace { message },
        sys::EID_ERR_HIP => AttnError::Hip { message },
        sys::EID_ERR_NO_BLOCKS => AttnError::NoBlocks { message },
        code => AttnError::Other { code, message },
    })
}

/// `(major, minor)` of the loaded library.
pub fn version() -> (u32, u32) {
    // SAFETY: no arguments, no state.
    let v = unsafe { sys::eid_version() };
    (v >> 16, v & 0xffff)
}

/// Storage type of the paged KV cache.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum KvDtype {
    Bf16,
    Fp8E4m3,
}

/// Model-side constants of an attention layer (gpt-oss: 64 query heads, 8 KV heads, head
/// dimension 64, 16-token pages).
#[derive(Clone, Copy, Debug)]
pub struct Geometry {
    pub num_q_heads: i32,
    pub num_kv_heads: i32,
    pub head_dim: i32,
    pub block_size: i32,
    pub softmax_scale: f32,
    /// 0 = full causal attention; W > 0: a row at position p sees p-W+1..=p.
    pub window: i32,
    pub kv_dtype: KvDtype,
    /// Split-KV partition in tokens (multiple of 64 in 64..=4096), 0 = sized at run time.
    pub partition_size: i32,
}

impl Default for Geometry {
    fn default() -> Self {
        Geometry {
            num_q_heads: 64,
            num_kv_heads: 8,
            head_dim: 64,
            block_size: 16,
            softmax_scale: 0.125,
            window: 0,
            kv_dtype: KvDtype::Bf16,
            partition_size: 0,
        }
    }
}

/// Shape of one batch: what `Scheduler::build_batch` reports, plus the pool's extent.
#[derive(Clone, Copy, Debug)]
pub struct BatchShape {
    pub num_seqs: i32,
    pub num_q_tokens: i32,
    pub max_q_len: i32,
    pub max_kv_len: i32,
    pub max_blocks_per_seq: i32,
    pub num_blocks: i64,
    /// Any value >= the sum of the sequences' KV lengths, or 0 when not known.
    pub sum_kv_len: i64,
}

/// Fills the C descriptor for a geometry and a batch.
pub fn descriptor(g: &Geometry, b: &BatchShape) -> sys::eid_attn_desc {
    sys::eid_attn_desc {
        struct_size: size_of::<sys::eid_attn_desc>() as u32,
        num_seqs: b.num_seqs,
        num_q_tokens: b.num_q_tokens,
        max_q_len: b.max_q_len,
        max_kv_len: b.max_kv_len,
        num_q_heads: g.num_q_heads,
        num_kv_heads: g.num_kv_heads,
        head_dim: g.head_dim,
        block_size: g.block_size,
        max_blocks_per_seq: b.max_blocks_per_seq,
        num_blocks: b.num_blocks,
        softmax_scale: g.softmax_scale,
        window: g.window,
        kv_dtype: match g.kv_dtype {
            KvDtype::Bf16 => sys::EID_KV_BF16,
            KvDtype::Fp8E4m3 => sys::EID_KV_FP8_E4M3,
        },
        partition_size: g.partition_size,
        sum_kv_len: b.sum_kv_len,
    }
}

/// Bytes of split-KV workspace the attention entry points need for this descriptor.
pub fn workspace_bytes(desc: &sys::eid_attn_desc) -> usize {
    // SAFETY: reads the descriptor only.
    unsafe { sys::eid_workspace_bytes(desc) }
}

/// Partition size (tokens) the workspace is planned with.
pub fn partition_size(desc: &sys::eid_attn_desc) -> i32 {
    // SAFETY: reads the descriptor only.
    unsafe { sys::eid_partition_size(desc) }
}

/// Device and host pointers of one attention call; the device memory is the caller's.
///
/// `None` host slices leave the planning to the kernels; given, they must equal the device
/// arrays (`EID_DEBUG=1` in the environment makes the library verify that).
pub struct AttnBuffers<'a> {
    pub q: *const c_void,
    pub out: *mut c_void,
    pub lse: Option<*mut f32>,
    pub k_cache: *mut c_void,
    pub v_cache: *mut c_void,
    pub block_table: *const i32,
    pub cu_seqlens_q: Option<*const i32>,
    pub seq_lens: *const i32,
    pub sinks: Option<*const f32>,
    pub k_scale: Option<*const f32>,
    pub v_scale: Option<*const f32>,
    pub workspace: *mut c_void,
    pub workspace_bytes: usize,
    /// Decode only: bf16 rows of every sequence's newest token, written into the cache by
    /// the call itself (both or neither).
    pub k_new: Option<*const c_void>,
    pub v_new: Option<*const c_void>,
    pub seq_lens_host: Option<&'a [i32]>,
    pub cu_seqlens_q_host: Option<&'a [i32]>,
    pub block_table_host: Option<&'a [i32]>,
}

impl AttnBuffers<'_> {
    fn raw(&self) -> sys::eid_attn_args {
        sys::eid_attn_args {
            q: self.q,
            out: self.out,
            lse: self.lse.unwrap_or(ptr::null_mut()),
            k_cache: self.k_cache,
            v_cache: self.v_cache,
            block_table: self.block_table,
            cu_seqlens_q: self.cu_seqlens_q.unwrap_or(ptr::null()),
            seq_lens: self.seq_lens,
            sinks: self.sinks.unwrap_or(ptr::null()),
            k_scale: self.k_scale.unwrap_or(ptr::null()),
            v_scale: self.v_scale.unwrap_or(ptr::null()),
            workspace: self.workspace,
            workspace_bytes: self.workspace_bytes,
            split_done_event: ptr::null_mut(),
            k_new: self.k_new.unwrap_or(ptr::null()),
            v_new: self.v_new.unwrap_or(ptr::null()),
            seq_lens_host: self.seq_lens_host.map_or(ptr::null(), |s| s.as_ptr()),
            cu_seqlens_q_host: self.cu_seqlens_q_host.map_or(ptr::null(), |s| s.as_ptr()),
            block_table_host: self.block_table_host.map_or(ptr::null(), |s| s.as_ptr()),
        }
    }
}

/// Slot-mapped KV-cache write of `num_tokens` new rows.
///
/// # Safety
/// Every pointer is a HIP device pointer of the extent `include/eidola_attn.h` states for
/// `eid_kv_write`; `stream` is a live `hipStream_t` (or null for the default stream); the
/// memory stays valid until the stream has passed the launch.
pub unsafe fn kv_write(
    desc: &sys::eid_attn_desc,
    k_new: *const c_void,
    v_new: *const c_void,
    k_cache: *mut c_void,
    v_cache: *mut c_void,
    slot_mapping: *const i64,
    num_tokens: i32,
    k_scale: Option<*const f32>,
    v_scale: Option<*const f32>,
    stream: *mut c_void,
) -> Result<(), AttnError> {
    check(unsafe {
        sys::eid_kv_write(
            desc,
            k_new,
            v_new,
            k_cache,
            v_cache,
            slot_mapping,
            num_tokens,
            k_scale.unwrap_or(ptr::null()),
            v_scale.unwrap_or(ptr::null()),
            stream,
        )
    })
}

/// Decode step: one query row per sequence (split-KV kernel + LSE merge).
///
/// # Safety
/// As `kv_write`, for the buffers of `eid_attn_decode`.
pub unsafe fn attn_decode(
    desc: &sys::eid_attn_desc,
    bufs: &AttnBuffers<'_>,
    stream: *mut c_void,
) -> Result<(), AttnError> {
    let args = bufs.raw();
    check(unsafe { sys::eid_attn_decode(desc, &args, stream) })
}

/// Decode step that allocates nothing and needs no workspace of the caller's: the partials
/// live in a static device array of `EID_STATIC_WORKSPACE_BYTES` inside the library.  Calls
/// that overlap on one GPU race on that array.
///
/// # Safety
/// As `attn_decode`; `bufs.workspace` is ignored.
pub unsafe fn attn_decode_noalloc(
    desc: &sys::eid_attn_desc,
    bufs: &AttnBuffers<'_>,
    stream: *mut c_void,
) -> Result<(), AttnError> {
    let args = bufs.raw();
    check(unsafe { sys::eid_attn_decode_noalloc(desc, &args, stream) })
}

/// Ragged batch: decode rows, verify rows and chunked-prefill rows in one call.
///
/// # Safety
/// As `attn_decode`, for the buffers of `eid_attn_varlen` (`cu_seqlens_q` is required).
pub unsafe fn attn_varlen(
    desc: &sys::eid_attn_desc,
    bufs: &AttnBuffers<'_>,
    stream: *mut c_void,
) -> Result<(), AttnError> {
    let args = bufs.raw();
    check(unsafe { sys::eid_attn_varlen(desc, &args, stream) })
}

/// The cross-partition merge by itself, over partials a split-KV launch left in the workspace.
///
/// # Safety
/// As `attn_decode`.
pub unsafe fn lse_merge(
    desc: &sys::eid_attn_desc,
    bufs: &AttnBuffers<'_>,
    stream: *mut c_void,
) -> Result<(), AttnError> {
    let args = bufs.raw();
    check(unsafe { sys::eid_lse_merge(desc, &args, stream) })
}

/// Output projection of the attention rows: `out = attn_out · weightᵀ (+ bias) (+ residual)`.
///
/// # Safety
/// Device pointers of the extents `eid_o_proj` states.
pub unsafe fn o_proj(
    attn_out: *const c_void,
    weight: *const c_void,
    bias: Option<*const c_void>,
    residual: Option<*const c_void>,
    out: *mut c_void,
    num_tokens: i32,
    out_features: i32,
    in_features: i32,
    stream: *mut c_void,
) -> Result<(), AttnError> {
    check(unsafe {
        sys::eid_o_proj(
            attn_out,
            weight,
            bias.unwrap_or(ptr::null()),
            residual.unwrap_or(ptr::null()),
            out,
            num_tokens,
            out_features,
            in_features,
            stream,
        )
    })
}

/// Arrays and scalars of one step, as `Scheduler::build_batch` fills them (host memory).
#[derive(Clone, Debug, Default)]
pub struct Batch {
    pub block_table: Vec<i32>,
    pub slot_mapping: Vec<i64>,
    pub cu_seqlens_q: Vec<i32>,
    pub seq_lens: Vec<i32>,
    pub positions: Vec<i32>,
    pub num_seqs: i32,
    pub num_q_tokens: i32,
    pub max_q_len: i32,
    pub max_kv_len: i32,
    pub sum_kv_len: i64,
}

/// The paged-KV block allocator and batch builder (`include/eidola_sched.h`).  Pure host state.
pub struct Scheduler {
    handle: *mut sys::eid_sched,
    max_blocks_per_seq: i32,
}

// The handle is a heap object with no thread affinity; calls need `&mut self` or are reads.
unsafe impl Send for Scheduler {}

impl Scheduler {
    pub fn new(
        num_blocks: i64,
        max_blocks_per_seq: i32,
        block_size: i32,
        prefix_reuse: bool,
    ) -> Result<Self, AttnError> {
        let cfg = sys::eid_sched_config {
            struct_size: size_of::<sys::eid_sched_config>() as u32,
            block_size,
            num_blocks,
            max_blocks_per_seq,
            prefix_reuse: prefix_reuse as i32,
        };
        let mut handle = ptr::null_mut();
        // SAFETY: cfg and handle outlive the call.
        check(unsafe { sys::eid_sched_create(&cfg, &mut handle) })?;
        Ok(Scheduler { handle, max_blocks_per_seq })
    }

    /// Registers a sequence; returns how many prompt tokens are already in the cache.
    pub fn add_seq(&mut self, seq_id: i64, prompt: Option<&[i32]>) -> Result<i32, AttnError> {
        let mut cached = 0i32;
        let (p, n) = prompt.map_or((ptr::null(), 0), |p| (p.as_ptr(), p.len() as i32));
        // SAFETY: the slice outlives the call; the library copies what it keeps.
        check(unsafe { sys::eid_sched_add_seq(self.handle, seq_id, p, n, &mut cached) })?;
        Ok(cached)
    }

    pub fn free_seq(&mut self, seq_id: i64) -> Result<(), AttnError> {
        // SAFETY: live handle.
        check(unsafe { sys::eid_sched_free_seq(self.handle, seq_id) })
    }

    /// Tokens in the cache for `seq_id`, `None` if the sequence is unknown.
    pub fn seq_len(&self, seq_id: i64) -> Option<i32> {
        // SAFETY: live handle.
        let n = unsafe { sys::eid_sched_seq_len(self.handle, seq_id) };
        (n >= 0).then_some(n)
    }

    pub fn free_blocks(&self) -> i64 {
        // SAFETY: live handle.
        unsafe { sys::eid_sched_free_blocks(self.handle) }
    }

    /// Reserves KV slots for `q_lens[i]` new tokens of `seq_ids[i]` and fills the step's arrays.
    /// All or nothing: on `AttnError::NoBlocks` no sequence has changed.
    pub fn build_batch(
        &mut self,
        seq_ids: &[i64],
        q_lens: &[i32],
        new_tokens: Option<&[i32]>,
    ) -> Result<Batch, AttnError> {
        if seq_ids.len() != q_lens.len() {
            return Err(AttnError::InvalidArg {
                message: "seq_ids and q_lens must be of equal length".into(),
            });
        }
        let num_seqs = seq_ids.len();
        let tokens: usize = q_lens.iter().map(|&q| q.max(0) as usize).sum();
        if new_tokens.is_some_and(|t| t.len() != tokens) {
            return Err(AttnError::InvalidArg {
                message: "new_tokens must hold one id per new token".into(),
            });
        }
        let mut b = Batch {
            block_table: vec![0; num_seqs * self.max_blocks_per_seq as usize],
            slot_mapping: vec![0; tokens],
            cu_seqlens_q: vec![0; num_seqs + 1],
            seq_lens: vec![0; num_seqs],
            positions: vec![0; tokens],
            ..Batch::default()
        };
        let mut info = sys::eid_batch_info::default();
        // SAFETY: every output vector has the extent the header states for it.
        check(unsafe {
            sys::eid_sched_build_batch(
                self.handle,
                seq_ids.as_ptr(),
                q_lens.as_ptr(),
                num_seqs as i32,
                new_tokens.map_or(ptr::null(), |t| t.as_ptr()),
                b.block_table.as_mut_ptr(),
                b.slot_mapping.as_mut_ptr(),
                b.cu_seqlens_q.as_mut_ptr(),
                b.seq_lens.as_mut_ptr(),
                b.positions.as_mut_ptr(),
                &mut info,
            )
        })?;
        b.num_seqs = info.num_seqs;
        b.num_q_tokens = info.num_q_tokens;
        b.max_q_len = info.max_q_len;
        b.max_kv_len = info.max_kv_len;
        b.sum_kv_len = info.sum_kv_len;
        Ok(b)
    }
}

impl Drop for Scheduler {
    fn drop(&mut self) {
        // SAFETY: created by eid_sched_create, destroyed once.
        unsafe { sys::eid_sched_destroy(self.handle) }
    }
}
