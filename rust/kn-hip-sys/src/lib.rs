//! `kn-hip-sys`: the C ABI of libknhip (`include/knhip.h`) and thin safe wrappers over its runtime tier, in the
//! shape of `kn-cuda-sys/src/wrapper` (handle.rs, event.rs, mem/device.rs, mem/pinned.rs, status.rs, group.rs).
//!
//! The graph builder entry points of the header (`knhip_graph_input`, ...) are not bound: on the Rust side the graph
//! is built by `kn-graph` and crosses the boundary serialised (`knhip_executor_new_from_blob`).
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

pub mod wrapper;

#[repr(C)]
pub struct knhip_executor {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Debug, Default, Copy, Clone)]
pub struct knhip_mem_usage {
    pub dedicated_bytes: usize,
    pub shared_bytes: usize,
    pub zero_bytes: usize,
    pub hypo_shared_bytes_peak: usize,
    pub hypo_shared_bytes_total: usize,
    pub arena_bytes: usize,
}

#[repr(C)]
#[derive(Debug, Default, Copy, Clone)]
pub struct knhip_profile {
    /// seconds per step kind: conv, mat_mul, scalar_op, reduce_op, softmax_op, layernorm_op, gather_op
    pub per_kind: [f32; 7],
    pub total_cpu: f32,
    pub total_gpu: f32,
    pub timing_overhead: f32,
    pub step_count: usize,
}

#[repr(C)]
#[derive(Debug, Copy, Clone)]
pub struct knhip_matmul_args {
    pub dtype: c_int,
    pub batch: c_int,
    pub m: c_int,
    pub n: c_int,
    pub k: c_int,
    pub a: *const c_void,
    pub a_batch_stride: i64,
    pub a_row_stride: i64,
    pub a_col_stride: i64,
    pub b: *const c_void,
    pub b_batch_stride: i64,
    pub b_row_stride: i64,
    pub b_col_stride: i64,
    pub c: *mut c_void,
    pub c_batch_stride: i64,
    pub c_row_stride: i64,
    pub c_col_stride: i64,
}

pub const KNHIP_OK: c_int = 0;
pub const KNHIP_ERROR: c_int = 1;
pub const KNHIP_BUFFER_TOO_SMALL: c_int = 2;

pub const KNHIP_PLAN_ONLY: c_int = 1;
pub const KNHIP_PRESERVE_INPUTS: c_int = 2;
pub const KNHIP_STEP_BY_STEP: c_int = 4;

pub const KNHIP_PROBE_NORMAL: c_int = 1;
pub const KNHIP_PROBE_F32: c_int = 2;
pub const KNHIP_PROBE_RECTIFIED: c_int = 4;

pub const KNHIP_F32: c_int = 0;
pub const KNHIP_F64: c_int = 1;
pub const KNHIP_I8: c_int = 2;
pub const KNHIP_I16: c_int = 3;
pub const KNHIP_I32: c_int = 4;
pub const KNHIP_I64: c_int = 5;
pub const KNHIP_U8: c_int = 6;
pub const KNHIP_U16: c_int = 7;
pub const KNHIP_U32: c_int = 8;
pub const KNHIP_U64: c_int = 9;
pub const KNHIP_BOOL: c_int = 10;
pub const KNHIP_F16: c_int = 11;

pub const KNHIP_STATIC_SCRATCH_BYTES: usize = 32 << 20;

extern "C" {
    pub fn knhip_last_error() -> *const c_char;

    // device and memory
    pub fn knhip_device_count(count: *mut c_int) -> c_int;
    pub fn knhip_device_name(device: c_int, buf: *mut c_char, cap: usize, needed: *mut usize) -> c_int;
    pub fn knhip_malloc(device: c_int, bytes: usize, ptr: *mut *mut c_void) -> c_int;
    pub fn knhip_free(device: c_int, ptr: *mut c_void) -> c_int;
    pub fn knhip_memcpy_h2d(device: c_int, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn knhip_memcpy_d2h(device: c_int, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn knhip_memcpy_d2d(device: c_int, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn knhip_host_alloc(bytes: usize, ptr: *mut *mut c_void) -> c_int;
    pub fn knhip_host_free(ptr: *mut c_void) -> c_int;
    pub fn knhip_device_synchronize(device: c_int) -> c_int;
    pub fn knhip_device_mfma_probe(device: c_int, mode: c_int, iterations: c_int, tflops: *mut f64, shader_mhz: *mut f64) -> c_int;

    // streams, events, asynchronous copies
    pub fn knhip_stream_create(device: c_int, stream: *mut *mut c_void) -> c_int;
    pub fn knhip_stream_destroy(device: c_int, stream: *mut c_void) -> c_int;
    pub fn knhip_stream_synchronize(device: c_int, stream: *mut c_void) -> c_int;
    pub fn knhip_stream_wait_event(device: c_int, stream: *mut c_void, event: *mut c_void) -> c_int;
    pub fn knhip_event_create(device: c_int, event: *mut *mut c_void) -> c_int;
    pub fn knhip_event_destroy(device: c_int, event: *mut c_void) -> c_int;
    pub fn knhip_event_record(device: c_int, event: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn knhip_event_synchronize(device: c_int, event: *mut c_void) -> c_int;
    pub fn knhip_event_elapsed_seconds(device: c_int, start: *mut c_void, end: *mut c_void, seconds: *mut f32) -> c_int;
    pub fn knhip_memcpy_h2d_async(device: c_int, dst: *mut c_void, src: *const c_void, bytes: usize, stream: *mut c_void) -> c_int;
    pub fn knhip_memcpy_d2h_async(device: c_int, dst: *mut c_void, src: *const c_void, bytes: usize, stream: *mut c_void) -> c_int;
    pub fn knhip_memcpy_d2d_async(device: c_int, dst: *mut c_void, src: *const c_void, bytes: usize, stream: *mut c_void) -> c_int;

    // the stand-alone batched matrix product
    pub fn knhip_batched_mat_mul_workspace_bytes(args: *const knhip_matmul_args, bytes: *mut usize) -> c_int;
    pub fn knhip_batched_mat_mul(device: c_int, stream: *mut c_void, args: *const knhip_matmul_args, workspace: *mut c_void,
                                 workspace_bytes: usize) -> c_int;
    pub fn knhip_batched_mat_mul_static(device: c_int, stream: *mut c_void, args: *const knhip_matmul_args) -> c_int;

    // executor
    pub fn knhip_executor_new_from_blob(device: c_int, blob: *const u8, len: usize, batch_size: usize, flags: c_int,
                                        out: *mut *mut knhip_executor) -> c_int;
    pub fn knhip_executor_free(ex: *mut knhip_executor);
    pub fn knhip_executor_io_count(ex: *const knhip_executor, inputs: *mut usize, outputs: *mut usize) -> c_int;
    pub fn knhip_executor_io_info(ex: *const knhip_executor, is_output: c_int, index: usize, dtype: *mut c_int, rank: *mut usize,
                                  dims: *mut usize, cap: usize) -> c_int;
    pub fn knhip_executor_evaluate(ex: *mut knhip_executor, inputs: *const *const c_void, input_bytes: *const usize,
                                   input_count: usize, outputs: *const *mut c_void, output_bytes: *const usize,
                                   output_count: usize) -> c_int;
    pub fn knhip_executor_run_async(ex: *mut knhip_executor) -> c_int;
    pub fn knhip_executor_set_graph_mode(ex: *mut knhip_executor, enabled: c_int) -> c_int;
    pub fn knhip_executor_synchronize(ex: *mut knhip_executor) -> c_int;
    pub fn knhip_executor_time_runs(ex: *mut knhip_executor, iterations: usize, elapsed_ms: *mut f32) -> c_int;
    pub fn knhip_executor_input_ptr(ex: *const knhip_executor, index: usize, ptr: *mut *mut c_void) -> c_int;
    pub fn knhip_executor_output_ptr(ex: *const knhip_executor, index: usize, ptr: *mut *mut c_void) -> c_int;
    pub fn knhip_executor_stream(ex: *const knhip_executor, stream: *mut *mut c_void) -> c_int;
    pub fn knhip_executor_set_profile(ex: *mut knhip_executor, enabled: c_int) -> c_int;
    pub fn knhip_executor_last_profile(ex: *const knhip_executor, available: *mut c_int, profile: *mut knhip_profile) -> c_int;
    pub fn knhip_executor_profile_step_seconds(ex: *const knhip_executor, buf: *mut f32, cap: usize) -> c_int;
    pub fn knhip_executor_profile_str(ex: *const knhip_executor, buf: *mut c_char, cap: usize, needed: *mut usize) -> c_int;
    pub fn knhip_executor_mem_usage(ex: *const knhip_executor, usage: *mut knhip_mem_usage) -> c_int;
    pub fn knhip_executor_step_count(ex: *const knhip_executor, count: *mut usize) -> c_int;
    pub fn knhip_executor_step_kind(ex: *const knhip_executor, index: usize, kind: *mut c_int) -> c_int;
    pub fn knhip_executor_step_str(ex: *const knhip_executor, index: usize, buf: *mut c_char, cap: usize, needed: *mut usize) -> c_int;
    pub fn knhip_executor_step_work(ex: *const knhip_executor, index: usize, flops: *mut f64, bytes: *mut f64) -> c_int;
    pub fn knhip_executor_fused_source(ex: *const knhip_executor, buf: *mut c_char, cap: usize, needed: *mut usize) -> c_int;
    pub fn knhip_executor_str(ex: *const knhip_executor, buf: *mut c_char, cap: usize, needed: *mut usize) -> c_int;

    pub fn knhip_compile_stats(compiled: *mut usize, memory_hits: *mut usize, disk_hits: *mut usize) -> c_int;
}
