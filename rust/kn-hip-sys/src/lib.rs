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

/// What an executor is built with beyond (device, graph, batch size); fill it with `knhip_executor_options_default`.
#[repr(C)]
#[derive(Debug, Copy, Clone)]
pub struct knhip_executor_options {
    pub struct_bytes: usize,
    pub plan_only: c_int,
    pub preserve_inputs: c_int,
    pub step_by_step: c_int,
    pub fuse_attention: c_int,
    pub fuse_gated_matmul: c_int,
    pub group_matmuls: c_int,
    pub pack_matmul_constants: c_int,
    pub pointwise_conv_as_matmul: c_int,
    pub join_elementwise: c_int,
    pub split_reduce: c_int,
    pub tiled_transpose: c_int,
    pub split_conv_channels: c_int,
    pub plane_conv_any_width: c_int,
    pub direct_gemm: c_int,
    pub split_k: c_int,
    pub tail_split: c_int,
    pub dot_products: c_int,
    pub streaming_bytes: u64,
    pub mapped_io_bytes: u64,
    pub stream_weights_bytes: u64,
}

/// A strided tensor in device memory that the caller owns (`DeviceTensor`); strides in elements.
#[repr(C)]
#[derive(Debug, Copy, Clone)]
pub struct knhip_tensor {
    pub ptr: *mut c_void,
    pub dtype: c_int,
    pub rank: usize,
    pub shape: *const usize,
    pub strides: *const i64,
}

#[repr(C)]
pub struct knhip_kernel {
    _private: [u8; 0],
}

pub const KNHIP_OK: c_int = 0;
pub const KNHIP_ERROR: c_int = 1;
pub const KNHIP_BUFFER_TOO_SMALL: c_int = 2;

pub const KNHIP_REDUCE_SUM: c_int = 0;
pub const KNHIP_REDUCE_MEAN: c_int = 1;
pub const KNHIP_REDUCE_PROD: c_int = 2;
pub const KNHIP_REDUCE_MAX: c_int = 3;
pub const KNHIP_REDUCE_MIN: c_int = 4;

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
    pub fn knhip_static_scratch_prepare(device: c_int) -> c_int;

    // device tensors and stand-alone kernels
    pub fn knhip_strided_copy(device: c_int, stream: *mut c_void, dst: *const knhip_tensor, src: *const knhip_tensor) -> c_int;
    pub fn knhip_scalar_kernel_new(device: c_int, operation: *const c_char, operands: *const knhip_tensor, operand_count: usize,
                                   out: *mut *mut knhip_kernel) -> c_int;
    pub fn knhip_reduce_kernel_new(device: c_int, reduce_op: c_int, input: *const knhip_tensor, output: *const knhip_tensor,
                                   axes: *const usize, axis_count: usize, out: *mut *mut knhip_kernel) -> c_int;
    pub fn knhip_softmax_kernel_new(device: c_int, input: *const knhip_tensor, output: *const knhip_tensor, axis: usize,
                                    input_scale: f32, out: *mut *mut knhip_kernel) -> c_int;
    pub fn knhip_layernorm_kernel_new(device: c_int, input: *const knhip_tensor, output: *const knhip_tensor, axis: usize, eps: f32,
                                      alpha0: f32, alpha1: f32, beta: f32, out: *mut *mut knhip_kernel) -> c_int;
    pub fn knhip_gather_kernel_new(device: c_int, input: *const knhip_tensor, indices: *const knhip_tensor,
                                   output: *const knhip_tensor, axis: usize, out: *mut *mut knhip_kernel) -> c_int;
    pub fn knhip_kernel_run(kernel: *const knhip_kernel, stream: *mut c_void, ptrs: *const *mut c_void, count: usize) -> c_int;
    pub fn knhip_kernel_info(kernel: *const knhip_kernel, strategy: *mut c_char, cap: usize, needed: *mut usize, grid: *mut u32,
                             block: *mut u32) -> c_int;
    pub fn knhip_kernel_free(kernel: *mut knhip_kernel);

    // layout algebra (kn-cuda-eval/src/shape.rs:25-285), computed by the library
    pub fn knhip_strided_flags(shape: *const usize, strides: *const i64, rank: usize, simple: *mut c_int, dense: *mut c_int) -> c_int;
    pub fn knhip_strided_view(shape: *const usize, strides: *const i64, rank: usize, new_shape: *const usize, new_rank: usize,
                              ok: *mut c_int, new_strides: *mut i64) -> c_int;
    pub fn knhip_strided_slice(shape: *const usize, strides: *const i64, rank: usize, axis: usize, start: usize, end: usize,
                               step: usize, out_shape: *mut usize, out_strides: *mut i64) -> c_int;

    // executor
    pub fn knhip_executor_options_default(options: *mut knhip_executor_options) -> c_int;
    pub fn knhip_executor_new_from_blob(device: c_int, blob: *const u8, len: usize, batch_size: usize,
                                        options: *const knhip_executor_options, out: *mut *mut knhip_executor) -> c_int;
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
