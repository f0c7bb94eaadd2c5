//! `HipExecutor`: `CudaExecutor` (kn-cuda-eval/src/executor.rs:20-266) on libknhip.
use std::fmt::{Debug, Display, Formatter};
use std::os::raw::{c_int, c_void};
use std::ptr::null_mut;

use kn_graph::dispatch_dtype;
use kn_graph::dtype::{DBool, DTensor, DType, Tensor};
use kn_graph::graph::Graph;
use kn_hip_sys::wrapper::{read_string, DevicePtr, ExecutorOptions, HipDevice, HipStream, Status};
use kn_hip_sys::*;

use crate::device_tensor::DeviceTensor;
use crate::serialize::{dtype_from_code, serialize_graph};
use crate::shape::StridedShape;

/// planner.rs:67-81, plus the size of the one arena every buffer lives in.
#[derive(Debug, Clone, Copy)]
pub struct MemoryUsage {
    pub dedicated_bytes: usize,
    pub shared_bytes: usize,
    pub zero_bytes: usize,
    pub hypo_shared_bytes_peak: usize,
    pub hypo_shared_bytes_total: usize,
    pub arena_bytes: usize,
}

/// executor.rs:43-59
#[derive(Default, Debug, Clone)]
pub struct Profile {
    pub steps: Vec<String>,

    pub conv: f32,
    pub mat_mul: f32,
    pub scalar_op: f32,
    pub reduce_op: f32,
    pub softmax_op: f32,
    pub layernorm_op: f32,
    pub gather_op: f32,

    pub total_cpu: f32,
    pub total_gpu: f32,
    pub timing_overhead: f32,
}

pub struct HipExecutor {
    raw: *mut knhip_executor,
    stream: HipStream,

    /// the dense input and output tensors inside the executor's arena (executor.rs:26-27); they live as long as the
    /// executor does
    pub device_inputs: Vec<DeviceTensor>,
    pub device_outputs: Vec<DeviceTensor>,

    pub batch_size: usize,
    pub mem_usage: MemoryUsage,

    profile: bool,
    last_profile: Option<Profile>,
    tensor_outputs: Vec<DTensor>,
}

// executor.rs:41: used from one thread at a time (&mut self), may move between threads
unsafe impl Send for HipExecutor {}

fn io_tensors(device: HipDevice, raw: *const knhip_executor, is_output: bool, count: usize) -> Vec<DeviceTensor> {
    (0..count)
        .map(|index| unsafe {
            let mut dtype: c_int = 0;
            let mut rank = 0usize;
            let mut dims = [0usize; 16];
            knhip_executor_io_info(raw, is_output as c_int, index, &mut dtype, &mut rank, dims.as_mut_ptr(), dims.len()).unwrap();
            let mut ptr = null_mut();
            if is_output {
                knhip_executor_output_ptr(raw, index, &mut ptr).unwrap();
            } else {
                knhip_executor_input_ptr(raw, index, &mut ptr).unwrap();
            }
            let dtype = dtype_from_code(dtype);
            let shape = StridedShape::new_simple(dims[..rank].to_vec());
            let len_bytes = shape.size() * dtype.size().bytes();
            DeviceTensor::from_parts(DevicePtr::borrowed(device, ptr, len_bytes), shape, dtype)
        })
        .collect()
}

fn zeros_dtensor(dtype: DType, shape: &[usize]) -> DTensor {
    let shape = shape.to_vec();
    dispatch_dtype!(dtype, |_T, _fs, ft| ft(Tensor::zeros(shape)))
}

/// A dense copy when the tensor is not in standard layout, the tensor itself (a cheap Arc clone) otherwise.
fn as_standard_layout(tensor: &DTensor) -> DTensor {
    kn_graph::dispatch_dtensor!(tensor, |_T, f, inner| f(inner.as_standard_layout().into_owned().into_shared()))
}

fn dtensor_ptr(tensor: &DTensor) -> *const c_void {
    kn_graph::dispatch_dtensor!(tensor, |_T, _f, inner| inner.as_ptr() as *const c_void)
}

fn dtensor_ptr_mut(tensor: &mut DTensor) -> *mut c_void {
    // the output tensors are created by this executor and never shared before `evaluate` returns a borrow
    kn_graph::dispatch_dtensor!(tensor, |_T, _f, inner| inner.as_mut_ptr() as *mut c_void)
}

fn dtensor_bytes(tensor: &DTensor) -> usize {
    tensor.len() * tensor.dtype().size().bytes()
}

impl HipExecutor {
    /// `CudaExecutor::new` (executor.rs:61-110): plans the graph for one concrete batch size, allocates the arena,
    /// uploads the constants and compiles the kernels.
    pub fn new(device: HipDevice, graph: &Graph, batch_size: usize) -> Self {
        Self::new_with_options(device, graph, batch_size, &ExecutorOptions::default())
    }

    /// `options`: e.g. `ExecutorOptions::default().preserve_inputs()` for callers that write `device_inputs` once and
    /// call `run_async` many times, or `mapped_io_bytes = 0` for callers that read `device_outputs` after `evaluate`.
    pub fn new_with_options(device: HipDevice, graph: &Graph, batch_size: usize, options: &ExecutorOptions) -> Self {
        let blob = serialize_graph(graph);
        let mut raw = null_mut();
        unsafe { knhip_executor_new_from_blob(device.inner(), blob.as_ptr(), blob.len(), batch_size, &options.0, &mut raw) }.unwrap();

        let (mut input_count, mut output_count) = (0usize, 0usize);
        unsafe { knhip_executor_io_count(raw, &mut input_count, &mut output_count) }.unwrap();
        let device_inputs = io_tensors(device, raw, false, input_count);
        let device_outputs = io_tensors(device, raw, true, output_count);
        let tensor_outputs = device_outputs.iter().map(|t| zeros_dtensor(t.dtype(), t.strided_shape().shape())).collect();

        let mut usage = knhip_mem_usage::default();
        unsafe { knhip_executor_mem_usage(raw, &mut usage) }.unwrap();
        let mut stream = null_mut();
        unsafe { knhip_executor_stream(raw, &mut stream) }.unwrap();

        HipExecutor {
            raw,
            stream: unsafe { HipStream::borrowed(device, stream) },
            device_inputs,
            device_outputs,
            batch_size,
            mem_usage: MemoryUsage {
                dedicated_bytes: usage.dedicated_bytes,
                shared_bytes: usage.shared_bytes,
                zero_bytes: usage.zero_bytes,
                hypo_shared_bytes_peak: usage.hypo_shared_bytes_peak,
                hypo_shared_bytes_total: usage.hypo_shared_bytes_total,
                arena_bytes: usage.arena_bytes,
            },
            profile: false,
            last_profile: None,
            tensor_outputs,
        }
    }

    pub fn stream(&self) -> &HipStream {
        &self.stream
    }

    /// `CudaExecutor::evaluate` (executor.rs:117-195). The asserts keep the reference's messages; the library checks
    /// the same things again on its side of the boundary.
    pub fn evaluate(&mut self, inputs: &[DTensor]) -> &[DTensor] {
        assert_eq!(inputs.len(), self.device_inputs.len(), "Wrong input count");
        for (i, (input, io)) in inputs.iter().zip(&self.device_inputs).enumerate() {
            assert_eq!(input.shape(), io.strided_shape().shape(), "Wrong shape for input {}", i);
            assert_eq!(input.dtype(), io.dtype(), "Wrong dtype for input {}", i);
        }

        let dense: Vec<DTensor> = inputs.iter().map(as_standard_layout).collect();
        // bools travel as one byte each, 0 or 1: DBool is repr(transparent) over bool
        let in_ptrs: Vec<*const c_void> = dense.iter().map(dtensor_ptr).collect();
        let in_bytes: Vec<usize> = dense.iter().map(dtensor_bytes).collect();
        let out_bytes: Vec<usize> = self.tensor_outputs.iter().map(dtensor_bytes).collect();

        // bool outputs come back through a byte buffer so that a byte other than 0 / 1 never becomes a `bool`
        let mut bool_staging: Vec<Option<Vec<u8>>> =
            self.tensor_outputs.iter().map(|t| matches!(t, DTensor::Bool(_)).then(|| vec![0u8; t.len()])).collect();
        let out_ptrs: Vec<*mut c_void> = self
            .tensor_outputs
            .iter_mut()
            .zip(bool_staging.iter_mut())
            .map(|(tensor, staging)| match staging {
                Some(bytes) => bytes.as_mut_ptr() as *mut c_void,
                None => dtensor_ptr_mut(tensor),
            })
            .collect();

        unsafe {
            knhip_executor_evaluate(
                self.raw,
                in_ptrs.as_ptr(),
                in_bytes.as_ptr(),
                in_ptrs.len(),
                out_ptrs.as_ptr(),
                out_bytes.as_ptr(),
                out_ptrs.len(),
            )
        }
        .unwrap();

        for (tensor, staging) in self.tensor_outputs.iter_mut().zip(&bool_staging) {
            if let (DTensor::Bool(tensor), Some(bytes)) = (tensor, staging) {
                let mut fail = false;
                for (x, &y) in tensor.iter_mut().zip(bytes) {
                    *x = DBool(y != 0);
                    fail |= y > 1;
                }
                assert!(!fail);
            }
        }

        self.refresh_profile();
        &self.tensor_outputs
    }

    /// `run_async` (executor.rs:197-258): queues every step on the executor's stream; no synchronisation before or
    /// after, so make sure `device_inputs` are written and synchronise before reading `device_outputs`.
    pub unsafe fn run_async(&mut self) {
        knhip_executor_run_async(self.raw).unwrap();
        self.refresh_profile();
    }

    pub fn set_profile(&mut self, profile: bool) {
        self.profile = profile;
        unsafe { knhip_executor_set_profile(self.raw, profile as c_int) }.unwrap();
    }

    pub fn last_profile(&self) -> Option<&Profile> {
        self.last_profile.as_ref()
    }

    /// Replay the launch list as one HIP graph (no counterpart in the reference).
    pub fn set_graph_mode(&mut self, enabled: bool) {
        unsafe { knhip_executor_set_graph_mode(self.raw, enabled as c_int) }.unwrap();
    }

    pub fn step_count(&self) -> usize {
        let mut count = 0usize;
        unsafe { knhip_executor_step_count(self.raw, &mut count) }.unwrap();
        count
    }

    pub fn step_str(&self, index: usize) -> String {
        read_string(|buf, cap, needed| unsafe { knhip_executor_step_str(self.raw, index, buf, cap, needed) })
    }

    fn refresh_profile(&mut self) {
        if !self.profile {
            self.last_profile = None;
            return;
        }
        let mut available: c_int = 0;
        let mut p = knhip_profile::default();
        unsafe { knhip_executor_last_profile(self.raw, &mut available, &mut p) }.unwrap();
        if available == 0 {
            self.last_profile = None;
            return;
        }
        let mut seconds = vec![0f32; p.step_count];
        unsafe { knhip_executor_profile_step_seconds(self.raw, seconds.as_mut_ptr(), seconds.len()) }.unwrap();
        let steps = seconds
            .iter()
            .enumerate()
            .map(|(i, time)| format!("{: >4} time {:>10.4} ms, step {}", i, time * 1e3, self.step_str(i)))
            .collect();
        self.last_profile = Some(Profile {
            steps,
            conv: p.per_kind[0],
            mat_mul: p.per_kind[1],
            scalar_op: p.per_kind[2],
            reduce_op: p.per_kind[3],
            softmax_op: p.per_kind[4],
            layernorm_op: p.per_kind[5],
            gather_op: p.per_kind[6],
            total_cpu: p.total_cpu,
            total_gpu: p.total_gpu,
            timing_overhead: p.timing_overhead,
        });
    }
}

impl Drop for HipExecutor {
    fn drop(&mut self) {
        unsafe { knhip_executor_free(self.raw) }
    }
}

impl Debug for HipExecutor {
    fn fmt(&self, f: &mut Formatter<'_>) -> std::fmt::Result {
        // the library prints batch size, memory usage, inputs, outputs and steps (executor.rs:269-289)
        let text = read_string(|buf, cap, needed| unsafe { knhip_executor_str(self.raw, buf, cap, needed) });
        write!(f, "{}", text)
    }
}

impl Display for Profile {
    /// executor.rs:291-325
    fn fmt(&self, f: &mut Formatter<'_>) -> std::fmt::Result {
        write!(f, "Profile {{\n  steps: [\n")?;
        for step in &self.steps {
            writeln!(f, "    {}", step)?;
        }
        write!(f, "  ]\n\n")?;

        let total =
            self.conv + self.mat_mul + self.scalar_op + self.reduce_op + self.softmax_op + self.layernorm_op + self.gather_op;
        let mut line = |name, time: f32| writeln!(f, "  {} {:>10.4} ms  {:>4.2}", name, time * 1e3, time / total);

        line("Conv:      ", self.conv)?;
        line("Matmul:    ", self.mat_mul)?;
        line("Scalar:    ", self.scalar_op)?;
        line("Reduce:    ", self.reduce_op)?;
        line("Softmax:   ", self.softmax_op)?;
        line("Layernorm: ", self.layernorm_op)?;
        line("Gather:    ", self.gather_op)?;

        writeln!(f, "  ==============================")?;
        writeln!(f, "  Total GPU:  {:>10.4} ms", self.total_gpu * 1e3)?;
        writeln!(f, "  Total CPU:  {:>10.4} ms", self.total_cpu * 1e3)?;
        writeln!(f, "  Overhead:   {:>10.4} ms", self.timing_overhead * 1e3)?;

        writeln!(f, "}}")?;
        Ok(())
    }
}
