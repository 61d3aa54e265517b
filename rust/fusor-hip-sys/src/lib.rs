//! Raw bindings to `libfusor_hip` (`include/fusor_hip.h`): the MI355X attention backend that takes the
//! place of the WGPU arm of `fusor::Tensor::flash_attention`
//! (fusor-ml/fusor/src/composite/flash_attention.rs:52-73, fusor-ml/core/src/composite/flash_attention.rs:28-52).
//!
//! One item here per item of the header, same names, same order of fields and arguments.  Every function
//! returns a status (`FHIP_OK` = 0); `fhip_last_error()` is the thread-local text of the last failure.
#![allow(non_camel_case_types)]
#![no_std]

use core::ffi::{c_char, c_int, c_uint, c_void};

// ---- status ------------------------------------------------------------------------------------
pub const FHIP_OK: c_int = 0;
/// What the reference panics on: shapes, divisibility, null pointers.
pub const FHIP_ERR_INVALID_ARG: c_int = 1;
/// A valid request with no kernel (e.g. head_dim > 512).
pub const FHIP_ERR_UNSUPPORTED: c_int = 2;
/// A HIP runtime call failed (reference: `fusor::Error::Gpu`).
pub const FHIP_ERR_HIP: c_int = 3;
/// Workspace missing or smaller than `fhip_flash_attention_workspace_bytes` reports.
pub const FHIP_ERR_WORKSPACE: c_int = 4;

// ---- opaque handles ----------------------------------------------------------------------------
#[repr(C)]
pub struct fhip_device {
    _private: [u8; 0],
}
#[repr(C)]
pub struct fhip_stream {
    _private: [u8; 0],
}
#[repr(C)]
pub struct fhip_event {
    _private: [u8; 0],
}
#[repr(C)]
pub struct fhip_graph {
    _private: [u8; 0],
}
#[repr(C)]
pub struct fhip_kv_cache {
    _private: [u8; 0],
}

// ---- enums (C enums without negative values: `unsigned int`) ------------------------------------
/// Element types (reference: `DataTypeEnum`, fusor-ml/core/src/tensor.rs:110-134).
pub type fhip_dtype = c_uint;
pub const FHIP_F32: fhip_dtype = 0;
pub const FHIP_F16: fhip_dtype = 1;
pub const FHIP_BF16: fhip_dtype = 2;

/// Mask layout (reference: `enum MaskKind`, fusor flash_attention.rs:11-19).
pub type fhip_mask_kind = c_uint;
pub const FHIP_MASK_NONE: fhip_mask_kind = 0;
/// `[q_seq_len, kv_seq_len]`, shared by every (batch, head).
pub const FHIP_MASK_QK: fhip_mask_kind = 1;
/// `[batch, kv_seq_len]`, broadcast over heads and queries.
pub const FHIP_MASK_BATCH_KEY: fhip_mask_kind = 2;

pub type fhip_kernel_id = c_uint;
pub const FHIP_KERNEL_AUTO: fhip_kernel_id = 0;
pub const FHIP_KERNEL_GENERIC: fhip_kernel_id = 1;
pub const FHIP_KERNEL_PREFILL_MFMA: fhip_kernel_id = 2;
pub const FHIP_KERNEL_PREFILL_F32: fhip_kernel_id = 3;
pub const FHIP_KERNEL_DECODE_SPLITKV: fhip_kernel_id = 4;
pub const FHIP_KERNEL_PREFILL_MFMA_ROWS64: fhip_kernel_id = 5;

/// Size of the per-GPU array `fhip_flash_attention_noalloc` uses as its workspace.
pub const FHIP_NOALLOC_WORKSPACE_BYTES: usize = 32 << 20;
/// Most `rounds` `fhip_calibration_mfma` accepts (about a second of matrix work).
pub const FHIP_CALIBRATION_MFMA_MAX_ROUNDS: i32 = 2000000;
/// Number of companion mixes `fhip_calibration_issue` knows (0 .. this - 1).
pub const FHIP_CALIBRATION_ISSUE_MIXES: i32 = 13;

// ---- structs -----------------------------------------------------------------------------------
/// Rank-4 strided view `[batch, heads, seq, head_dim]`; offset and strides in elements
/// (fusor-ml/types/src/layout.rs:88-129).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fhip_tensor4 {
    pub ptr: *mut c_void,
    pub offset: u64,
    pub shape: [u32; 4],
    pub stride: [i64; 4],
}

/// Rank-2 strided view (the mask).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fhip_tensor2 {
    pub ptr: *mut c_void,
    pub offset: u64,
    pub shape: [u32; 2],
    pub stride: [i64; 2],
}

/// The mask `MaskCache::get_mask` builds, as a formula (fusor-ml/fusor/src/cache/mask_cache.rs:36-116).
#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq, Eq)]
pub struct fhip_analytic_mask {
    pub enabled: i32,
    pub causal: i32,
    pub q_pos_offset: i64,
    pub window: i64,
}

/// Arguments of one attention call.  Zero-initialise (`core::mem::zeroed`), then fill.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fhip_attn_args {
    pub q: fhip_tensor4,
    pub k: fhip_tensor4,
    pub v: fhip_tensor4,
    pub out: fhip_tensor4,
    pub dtype: fhip_dtype,
    pub out_dtype: fhip_dtype,
    pub scale: f32,
    pub mask_kind: fhip_mask_kind,
    pub mask: fhip_tensor2,
    pub analytic: fhip_analytic_mask,
    pub kv_lens: *const i32,
    pub workspace: *mut c_void,
    pub workspace_bytes: usize,
    pub force_kernel: i32,
    pub main_kernel_done: *mut fhip_event,
    pub main_kernel_start: *mut fhip_event,
    pub mask_intervals: *const c_void,
}

/// How a call would run on the split-KV decode kernels (`fhip_flash_attention_decode_plan`).
#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq, Eq)]
pub struct fhip_decode_plan_info {
    pub is_decode: i32,
    pub nsplit: i32,
    pub chunk: i32,
    pub wavefronts: i32,
    pub kernels: i32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct fhip_device_info {
    pub name: [c_char; 128],
    pub arch: [c_char; 64],
    pub compute_units: i32,
    pub wavefront_size: i32,
    pub clock_khz: i32,
    pub memory_clock_khz: i32,
    pub memory_bus_bits: i32,
    pub total_memory: u64,
    pub lds_per_cu: u64,
    pub l2_bytes: u64,
}

/// `RopeCache`'s tables on the device (fusor-ml/fusor/src/composite/rope.rs:180-265).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fhip_rope_tables {
    pub cos: *const f32,
    pub sin: *const f32,
    pub table_rows: u64,
    pub start_pos: u64,
    pub interleaved: i32,
}

/// An `RmsNorm`'s device parameters (fusor-ml/fusor/src/layers/rms_norm.rs:122-133).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct fhip_rms_norm {
    pub weight: *const c_void,
    pub bias: *const c_void,
    pub dtype: fhip_dtype,
    pub eps: f32,
}

// ---- functions ---------------------------------------------------------------------------------
unsafe extern "C" {
    pub fn fhip_last_error() -> *const c_char;

    // device / stream / memory
    pub fn fhip_device_count(count: *mut i32) -> c_int;
    pub fn fhip_device_create(ordinal: i32, out: *mut *mut fhip_device) -> c_int;
    pub fn fhip_device_destroy(dev: *mut fhip_device) -> c_int;
    pub fn fhip_device_get_info(dev: *mut fhip_device, info: *mut fhip_device_info) -> c_int;

    pub fn fhip_stream_create(dev: *mut fhip_device, out: *mut *mut fhip_stream) -> c_int;
    pub fn fhip_stream_destroy(s: *mut fhip_stream) -> c_int;
    pub fn fhip_stream_synchronize(s: *mut fhip_stream) -> c_int;

    pub fn fhip_malloc(dev: *mut fhip_device, bytes: usize, out: *mut *mut c_void) -> c_int;
    pub fn fhip_free(dev: *mut fhip_device, ptr: *mut c_void) -> c_int;
    pub fn fhip_memcpy_h2d(s: *mut fhip_stream, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn fhip_memcpy_d2h(s: *mut fhip_stream, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn fhip_memcpy_d2d(s: *mut fhip_stream, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn fhip_memset(s: *mut fhip_stream, dst: *mut c_void, value: c_int, bytes: usize) -> c_int;

    // stream capture
    pub fn fhip_stream_begin_capture(s: *mut fhip_stream) -> c_int;
    pub fn fhip_stream_end_capture(s: *mut fhip_stream, out: *mut *mut fhip_graph) -> c_int;
    pub fn fhip_graph_launch(g: *mut fhip_graph, s: *mut fhip_stream) -> c_int;
    pub fn fhip_graph_destroy(g: *mut fhip_graph) -> c_int;

    // events
    pub fn fhip_event_create(dev: *mut fhip_device, out: *mut *mut fhip_event) -> c_int;
    pub fn fhip_event_destroy(e: *mut fhip_event) -> c_int;
    pub fn fhip_event_record(e: *mut fhip_event, s: *mut fhip_stream) -> c_int;
    pub fn fhip_event_synchronize(e: *mut fhip_event) -> c_int;
    pub fn fhip_event_elapsed_ms(start: *mut fhip_event, stop: *mut fhip_event, ms: *mut f32) -> c_int;

    // attention
    pub fn fhip_flash_attention_validate(args: *const fhip_attn_args) -> c_int;
    pub fn fhip_flash_attention_select(args: *const fhip_attn_args, kernel_id: *mut i32) -> c_int;
    pub fn fhip_flash_attention_workspace_bytes(
        args: *const fhip_attn_args,
        compute_units: i32,
        bytes: *mut usize,
    ) -> c_int;
    pub fn fhip_flash_attention_decode_plan(
        s: *mut fhip_stream,
        args: *const fhip_attn_args,
        info: *mut fhip_decode_plan_info,
    ) -> c_int;
    pub fn fhip_flash_attention(s: *mut fhip_stream, args: *const fhip_attn_args) -> c_int;
    pub fn fhip_flash_attention_noalloc(s: *mut fhip_stream, args: *const fhip_attn_args) -> c_int;

    // calibration for benchmarks: the register-only matrix-core loop
    pub fn fhip_calibration_mfma(
        s: *mut fhip_stream,
        dtype: fhip_dtype,
        random_operands: i32,
        duty_percent: i32,
        rounds: i32,
        scratch: *mut c_void,
        scratch_bytes: usize,
    ) -> c_int;

    pub fn fhip_calibration_issue(s: *mut fhip_stream, mix: i32, rounds: i32, scratch: *mut c_void, scratch_bytes: usize) -> c_int;
    pub fn fhip_calibration_xcd_map(s: *mut fhip_stream, workgroups: u32, out: *mut c_void, out_bytes: usize) -> c_int;
    pub fn fhip_calibration_read(
        s: *mut fhip_stream,
        src: *const c_void,
        bytes: usize,
        scratch: *mut c_void,
        scratch_bytes: usize,
    ) -> c_int;

    // masks
    pub fn fhip_mask_causal(dtype: fhip_dtype, seq_len: u32, out: *mut c_void) -> c_int;
    pub fn fhip_mask_sliding_window(dtype: fhip_dtype, seq_len: u32, window: u64, out: *mut c_void) -> c_int;
    pub fn fhip_mask_get_mask_shape(
        seq_len: u32,
        seqlen_offset: u64,
        has_window: i32,
        window: u64,
        rows: *mut u32,
        cols: *mut u64,
    ) -> c_int;
    pub fn fhip_mask_get_mask(
        dtype: fhip_dtype,
        seq_len: u32,
        seqlen_offset: u64,
        has_window: i32,
        window: u64,
        out: *mut c_void,
    ) -> c_int;
    pub fn fhip_mask_get_mask_device(
        s: *mut fhip_stream,
        dtype: fhip_dtype,
        seq_len: u32,
        seqlen_offset: u64,
        has_window: i32,
        window: u64,
        out_device: *mut c_void,
    ) -> c_int;
    pub fn fhip_mask_intervals_bytes(rows: u32, bytes: *mut usize) -> c_int;
    pub fn fhip_mask_intervals(
        s: *mut fhip_stream,
        mask: *const fhip_tensor2,
        dtype: fhip_dtype,
        table: *mut c_void,
        table_bytes: usize,
    ) -> c_int;
    pub fn fhip_mask_get_analytic(
        seq_len: u32,
        seqlen_offset: u64,
        has_window: i32,
        window: u64,
        out: *mut fhip_analytic_mask,
    ) -> c_int;

    // KV cache
    pub fn fhip_kv_cache_create(
        dev: *mut fhip_device,
        dtype: fhip_dtype,
        max_sequence_len: u64,
        out: *mut *mut fhip_kv_cache,
    ) -> c_int;
    pub fn fhip_kv_cache_destroy(c: *mut fhip_kv_cache) -> c_int;
    pub fn fhip_kv_cache_reset(c: *mut fhip_kv_cache) -> c_int;
    pub fn fhip_kv_cache_current_seq_len(c: *const fhip_kv_cache, len: *mut u64) -> c_int;
    pub fn fhip_kv_cache_allocated_seq_len(c: *const fhip_kv_cache, len: *mut u64) -> c_int;
    pub fn fhip_kv_cache_append(
        c: *mut fhip_kv_cache,
        s: *mut fhip_stream,
        k_new: *const fhip_tensor4,
        v_new: *const fhip_tensor4,
        k_all: *mut fhip_tensor4,
        v_all: *mut fhip_tensor4,
    ) -> c_int;

    // rotary embedding, q/k norm, fused cache writes
    pub fn fhip_rope(
        s: *mut fhip_stream,
        rope: *const fhip_rope_tables,
        x: *const fhip_tensor4,
        x_dtype: fhip_dtype,
        out: *const fhip_tensor4,
        out_dtype: fhip_dtype,
    ) -> c_int;
    pub fn fhip_kv_cache_rope_append(
        c: *mut fhip_kv_cache,
        s: *mut fhip_stream,
        rope: *const fhip_rope_tables,
        k_new: *const fhip_tensor4,
        v_new: *const fhip_tensor4,
        in_dtype: fhip_dtype,
        k_all: *mut fhip_tensor4,
        v_all: *mut fhip_tensor4,
    ) -> c_int;
    pub fn fhip_norm_rope(
        s: *mut fhip_stream,
        norm: *const fhip_rms_norm,
        rope: *const fhip_rope_tables,
        x: *const fhip_tensor4,
        x_dtype: fhip_dtype,
        out: *const fhip_tensor4,
        out_dtype: fhip_dtype,
    ) -> c_int;
    pub fn fhip_kv_cache_norm_rope_append(
        c: *mut fhip_kv_cache,
        s: *mut fhip_stream,
        k_norm: *const fhip_rms_norm,
        rope: *const fhip_rope_tables,
        k_new: *const fhip_tensor4,
        v_new: *const fhip_tensor4,
        in_dtype: fhip_dtype,
        k_all: *mut fhip_tensor4,
        v_all: *mut fhip_tensor4,
    ) -> c_int;
    pub fn fhip_kv_cache_qkv_rope_append(
        c: *mut fhip_kv_cache,
        s: *mut fhip_stream,
        q_norm: *const fhip_rms_norm,
        k_norm: *const fhip_rms_norm,
        rope: *const fhip_rope_tables,
        q: *const fhip_tensor4,
        q_dtype: fhip_dtype,
        q_out: *const fhip_tensor4,
        q_out_dtype: fhip_dtype,
        k_new: *const fhip_tensor4,
        v_new: *const fhip_tensor4,
        in_dtype: fhip_dtype,
        k_all: *mut fhip_tensor4,
        v_all: *mut fhip_tensor4,
    ) -> c_int;

    pub fn fhip_version() -> *const c_char;
}

// Layout checks the compiler runs: sizes the C side has on x86-64 / LP64.
const _: () = {
    assert!(core::mem::size_of::<fhip_tensor4>() == 64);
    assert!(core::mem::size_of::<fhip_tensor2>() == 40);
    assert!(core::mem::size_of::<fhip_analytic_mask>() == 24);
    assert!(core::mem::size_of::<fhip_attn_args>() == 392);
    assert!(core::mem::size_of::<fhip_device_info>() == 240);
    assert!(core::mem::size_of::<fhip_decode_plan_info>() == 20);
    assert!(core::mem::size_of::<fhip_rope_tables>() == 40);
    assert!(core::mem::size_of::<fhip_rms_norm>() == 24);
};
