//! The C ABI of liblng_hip.so, declaration for declaration as `include/lng_hip.h` has it.
//!
//! Every struct is `#[repr(C)]` with the header's fields in the header's order; every count is a
//! `u64`, every length of host memory a `usize` (`size_t`), every status an `i32` (`int`).
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

/// `LNG_WINDOW_FULL`: a query sees every earlier position.
pub const LNG_WINDOW_FULL: u64 = u64::MAX;
/// `LNG_NO_SINKS`: `LngDecodeItem::sinks_offset` of an item without sinks.
pub const LNG_NO_SINKS: u64 = u64::MAX;

pub const LNG_OK: c_int = 0;
pub const LNG_ERR_NO_DEVICE: c_int = -1;
pub const LNG_ERR_COMPILE: c_int = -2;
pub const LNG_ERR_ALLOC: c_int = -3;
pub const LNG_ERR_DISPATCH: c_int = -4;
pub const LNG_ERR_GPU: c_int = -5;

pub const LNG_F32: c_int = 0;
pub const LNG_BF16: c_int = 1;

pub const LNG_STATIC_SCRATCH_SLOTS: u32 = 65536;
pub const LNG_STATIC_MAX_ROW_HEADS: u32 = 2048;

/// `struct lng_gpu` (opaque).
#[repr(C)]
pub struct LngGpu {
    _opaque: [u8; 0],
}
/// `struct lng_buffer` (opaque): a buffer or a resident.
#[repr(C)]
pub struct LngBuffer {
    _opaque: [u8; 0],
}
/// `struct lng_batch` (opaque).
#[repr(C)]
pub struct LngBatch {
    _opaque: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct LngSlice {
    pub buffer: u64,
    pub offset: u64,
    pub len: u64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct LngGroupedShape {
    pub t: u64,
    pub start: u64,
    pub heads: u64,
    pub kv_heads: u64,
    pub dim: u64,
    pub window: u64,
    pub slots: u64,
    pub scale: f32,
}

#[repr(C)]
pub struct LngCompleted {
    pub status: c_int,
    pub gpu_seconds: f64,
    /// Valid during the callback only.
    pub message: *const c_char,
}

/// `lng_on_done`: runs once on a thread of the library when the GPU has finished the batch.
pub type LngOnDone = Option<unsafe extern "C" fn(done: *const LngCompleted, user: *mut c_void)>;

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct LngDecodeItem {
    pub q_offset: u64,
    pub out_offset: u64,
    pub k_offset: u64,
    pub v_offset: u64,
    pub sinks_offset: u64,
    pub start: u64,
    pub window: u64,
    pub slots: u64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct LngPrepareItem {
    pub q_offset: u64,
    pub k_offset: u64,
    pub v_offset: u64,
    pub table_offset: u64,
    pub q_out_offset: u64,
    pub k_cache_offset: u64,
    pub v_cache_offset: u64,
    pub n: u64,
    pub start: u64,
    pub slots: u64,
}

#[repr(C)]
pub struct LngPrepareBuffers {
    pub q: u64,
    pub k: u64,
    pub v: u64,
    pub table: u64,
    pub q_out: u64,
    pub k_cache: u64,
    pub v_cache: u64,
    pub q_bias: *const LngSlice,
    pub k_bias: *const LngSlice,
    pub v_bias: *const LngSlice,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct LngQ8Matrix {
    pub codes: LngSlice,
    pub scales: LngSlice,
    pub y: LngSlice,
    pub rows: u64,
}

extern "C" {
    pub fn lng_hip_last_error() -> *const c_char;

    // ---- device ----
    pub fn lng_hip_open(device: c_int, gpu: *mut *mut LngGpu) -> c_int;
    pub fn lng_hip_close(gpu: *mut LngGpu);
    pub fn lng_hip_device_name(gpu: *mut LngGpu, name: *mut c_char, cap: usize) -> c_int;
    /// Development switches (not part of the interface); `value` null puts the default back.
    pub fn lng_hip_debug_set(gpu: *mut LngGpu, name: *const c_char, value: *const c_char) -> c_int;
    /// Development counters (not part of the interface): read and reset.
    pub fn lng_hip_debug_get(gpu: *mut LngGpu, name: *const c_char, value: *mut u64) -> c_int;

    // ---- memory ----
    pub fn lng_hip_buffer(gpu: *mut LngGpu, len: usize, buffer: *mut *mut LngBuffer) -> c_int;
    pub fn lng_hip_resident(gpu: *mut LngGpu, bytes: *const c_void, len: usize, resident: *mut *mut LngBuffer) -> c_int;
    pub fn lng_hip_buffer_free(buffer: *mut LngBuffer) -> c_int;
    pub fn lng_hip_buffer_len(buffer: *const LngBuffer) -> usize;
    pub fn lng_hip_buffer_device_ptr(buffer: *mut LngBuffer) -> *mut c_void;
    pub fn lng_hip_upload(buffer: *mut LngBuffer, offset: usize, src: *const c_void, len: usize) -> c_int;
    pub fn lng_hip_download(buffer: *mut LngBuffer, offset: usize, dst: *mut c_void, len: usize) -> c_int;
    pub fn lng_hip_fill(buffer: *mut LngBuffer, offset: usize, byte: c_int, len: usize) -> c_int;

    // ---- batches ----
    pub fn lng_hip_batch(gpu: *mut LngGpu, buffers: *const *mut LngBuffer, n_buffers: usize, batch: *mut *mut LngBatch) -> c_int;
    pub fn lng_hip_batch_attach(batch: *mut LngBatch, resident: *mut LngBuffer, whole: *mut LngSlice) -> c_int;
    pub fn lng_hip_batch_dispatches(batch: *const LngBatch) -> usize;
    pub fn lng_hip_batch_barrier(batch: *mut LngBatch) -> c_int;
    pub fn lng_hip_batch_commit(batch: *mut LngBatch, on_done: LngOnDone, user: *mut c_void) -> c_int;
    pub fn lng_hip_batch_wait(batch: *mut LngBatch, gpu_seconds: *mut f64) -> c_int;
    pub fn lng_hip_batch_set_timing(batch: *mut LngBatch, enabled: c_int) -> c_int;
    pub fn lng_hip_batch_kernel_seconds(batch: *mut LngBatch, kernel: *const c_char, seconds: *mut f64, launches: *mut usize) -> c_int;
    pub fn lng_hip_batch_drop(batch: *mut LngBatch);

    // ---- the attention operator ----
    pub fn lng_hip_check_grouped(shape: *const LngGroupedShape, tiled: c_int) -> c_int;
    pub fn lng_hip_attention_grouped(
        batch: *mut LngBatch, q: LngSlice, k: LngSlice, v: LngSlice, out: LngSlice, sinks: *const LngSlice,
        shape: *const LngGroupedShape, dtype: c_int,
    ) -> c_int;
    pub fn lng_hip_attention_grouped_tiled(
        batch: *mut LngBatch, q: LngSlice, k: LngSlice, v: LngSlice, out: LngSlice, sinks: *const LngSlice,
        shape: *const LngGroupedShape, dtype: c_int,
    ) -> c_int;
    pub fn lng_hip_attention_grouped_static(
        gpu: *mut LngGpu, stream: *mut c_void, q: *const c_void, k: *const c_void, v: *const c_void, out: *mut c_void,
        sinks: *const f32, shape: *const LngGroupedShape, dtype: c_int,
    ) -> c_int;
    pub fn lng_hip_copy_rows(
        batch: *mut LngBatch, src: LngSlice, src_stride: u64, src_dtype: c_int, dst: LngSlice, dst_stride: u64,
        dst_dtype: c_int, rows: u64, width: u64,
    ) -> c_int;
    pub fn lng_hip_attention_decode_batched(
        batch: *mut LngBatch, q_buffer: u64, k_buffer: u64, v_buffer: u64, out_buffer: u64, sinks_buffer: u64,
        items: *const LngDecodeItem, n_items: usize, heads: u64, kv_heads: u64, dim: u64, scale: f32, dtype: c_int,
    ) -> c_int;

    // ---- the step before attention ----
    pub fn lng_hip_rmsnorm_rows(batch: *mut LngBatch, v: LngSlice, w: LngSlice, rows: u64, d: u64, stride: u64, eps: f32) -> c_int;
    pub fn lng_hip_add_rows(batch: *mut LngBatch, dst: LngSlice, src: LngSlice, src_stride: u64, rows: u64, width: u64) -> c_int;
    pub fn lng_hip_rotate_halves(batch: *mut LngBatch, x: LngSlice, table: LngSlice, rows: u64, heads: u64, dim: u64, rotary: u64) -> c_int;
    pub fn lng_hip_prepare_attention(
        batch: *mut LngBatch, buffers: *const LngPrepareBuffers, items: *const LngPrepareItem, n_items: usize, heads: u64,
        kv_heads: u64, dim: u64, rotary: u64, out_dtype: c_int,
    ) -> c_int;

    // ---- Q8_0 products ----
    pub fn lng_hip_gemv_q8_0(batch: *mut LngBatch, codes: LngSlice, scales: LngSlice, x: LngSlice, y: LngSlice, rows: u64, cols: u64) -> c_int;
    pub fn lng_hip_gemm_q8_0(
        batch: *mut LngBatch, codes: LngSlice, scales: LngSlice, x: LngSlice, y: LngSlice, rows: u64, cols: u64, n: u64,
        x_stride: u64, y_stride: u64,
    ) -> c_int;
    pub fn lng_hip_gemm_q8_0_tiled(
        batch: *mut LngBatch, codes: LngSlice, scales: LngSlice, x: LngSlice, y: LngSlice, rows: u64, cols: u64, n: u64,
        x_stride: u64, y_stride: u64,
    ) -> c_int;
    pub fn lng_hip_gemm_q8_0_bf16(
        batch: *mut LngBatch, codes: LngSlice, scales: LngSlice, x: LngSlice, y: LngSlice, rows: u64, cols: u64, n: u64,
        x_stride: u64, y_stride: u64,
    ) -> c_int;
    pub fn lng_hip_gemm_q8_0_many(
        batch: *mut LngBatch, matrices: *const LngQ8Matrix, n_matrices: usize, x: LngSlice, cols: u64, n: u64, x_stride: u64,
    ) -> c_int;
    pub fn lng_hip_gemm_q8_0_many_normed(
        batch: *mut LngBatch, matrices: *const LngQ8Matrix, n_matrices: usize, x: LngSlice, norm_w: LngSlice, eps: f32,
        cols: u64, n: u64, x_stride: u64,
    ) -> c_int;
    pub fn lng_hip_gemm_q8_0_residual(
        batch: *mut LngBatch, codes: LngSlice, scales: LngSlice, x: LngSlice, x_dtype: c_int, bias: *const LngSlice,
        h: LngSlice, rows: u64, cols: u64, n: u64, x_stride: u64, h_stride: u64,
    ) -> c_int;

    pub fn lng_hip_checksum(batch: *mut LngBatch, src: LngSlice, dst: LngSlice) -> c_int;
    pub fn lng_hip_fill_synthetic(batch: *mut LngBatch, dst: LngSlice, dtype: c_int, seed: u64, scale: f32, period: u64) -> c_int;
}
