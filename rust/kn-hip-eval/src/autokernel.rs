//! The run-time compiled kernels of kn-cuda-eval/src/autokernel/ on caller-owned tensors: `ScalarKernel`
//! (scalar.rs:33-154), `ReduceKernel` (reduce.rs:35-153), `SoftmaxKernel` (softmax.rs:28-108), `LayernormKernel`
//! (layernorm.rs:33-136), `GatherKernel` (gather.rs:30-129). The kernels are generated, compiled and cached by the
//! library; `run` checks the tensors against the shapes the kernel was built for, like the reference's asserts.
use std::ffi::CString;
use std::os::raw::{c_int, c_void};
use std::ptr::null_mut;

use kn_graph::dtype::DType;
use kn_graph::graph::ReduceOp;
use kn_hip_sys::wrapper::{HipDevice, HipStream, Status};
use kn_hip_sys::*;

use crate::device_tensor::DeviceTensor;
use crate::serialize::dtype_code;
use crate::shape::StridedShape;

struct Descriptor {
    raw: knhip_tensor,
    _shape: Vec<usize>,
    _strides: Vec<i64>,
}

fn describe(shape: &StridedShape, dtype: DType) -> Descriptor {
    let dims = shape.shape().to_vec();
    let strides = shape.strides_i64();
    let raw = knhip_tensor { ptr: null_mut(), dtype: dtype_code(dtype) as c_int, rank: dims.len(), shape: dims.as_ptr(), strides: strides.as_ptr() };
    Descriptor { raw, _shape: dims, _strides: strides }
}

#[derive(Debug)]
struct RawKernel(*mut knhip_kernel);

impl RawKernel {
    unsafe fn run(&self, stream: &HipStream, ptrs: &[*mut c_void]) {
        knhip_kernel_run(self.0, stream.inner(), ptrs.as_ptr(), ptrs.len()).unwrap()
    }
}

impl Drop for RawKernel {
    fn drop(&mut self) {
        unsafe { knhip_kernel_free(self.0) }
    }
}

fn reduce_code(op: ReduceOp) -> c_int {
    match op {
        ReduceOp::Sum => KNHIP_REDUCE_SUM,
        ReduceOp::Mean => KNHIP_REDUCE_MEAN,
        ReduceOp::Prod => KNHIP_REDUCE_PROD,
        ReduceOp::Max => KNHIP_REDUCE_MAX,
        ReduceOp::Min => KNHIP_REDUCE_MIN,
    }
}

#[derive(Debug)]
pub struct ScalarKernel {
    raw: RawKernel,
    shapes: Vec<StridedShape>,
    dtypes: Vec<DType>,
}

impl ScalarKernel {
    /// `operation` has the format `*x0 = *x1 + *x2;` (scalar.rs:36); operand 0 is written, the others are read.
    pub fn new_for_shapes(device: HipDevice, operation: &str, shapes: &[StridedShape], operand_types: Vec<DType>) -> Self {
        assert!(!shapes.is_empty());
        assert_eq!(shapes.len(), operand_types.len());
        let descriptors: Vec<Descriptor> = shapes.iter().zip(&operand_types).map(|(s, &t)| describe(s, t)).collect();
        let raws: Vec<knhip_tensor> = descriptors.iter().map(|d| d.raw).collect();
        let operation = CString::new(operation).unwrap();
        let mut raw = null_mut();
        unsafe { knhip_scalar_kernel_new(device.inner(), operation.as_ptr(), raws.as_ptr(), raws.len(), &mut raw) }.unwrap();
        ScalarKernel { raw: RawKernel(raw), shapes: shapes.to_vec(), dtypes: operand_types }
    }

    pub unsafe fn run(&self, stream: &HipStream, tensors: &[DeviceTensor]) {
        assert_eq!(tensors.len(), self.shapes.len());
        for ((tensor, shape), &dtype) in tensors.iter().zip(&self.shapes).zip(&self.dtypes) {
            assert_eq!(tensor.strided_shape(), shape);
            assert_eq!(tensor.dtype(), dtype);
        }
        let ptrs: Vec<*mut c_void> = tensors.iter().map(|t| t.ptr().ptr()).collect();
        self.raw.run(stream, &ptrs);
    }
}

#[derive(Debug)]
pub struct ReduceKernel {
    raw: RawKernel,
    input_shape: StridedShape,
    output_shape: StridedShape,
}

impl ReduceKernel {
    pub fn new(device: HipDevice, op: ReduceOp, dtype: DType, input_shape: &StridedShape, output_shape: &StridedShape, reduced_axes: &[usize]) -> Self {
        let (input, output) = (describe(input_shape, dtype), describe(output_shape, dtype));
        let mut raw = null_mut();
        unsafe {
            knhip_reduce_kernel_new(device.inner(), reduce_code(op), &input.raw, &output.raw, reduced_axes.as_ptr(), reduced_axes.len(), &mut raw)
        }
        .unwrap();
        ReduceKernel { raw: RawKernel(raw), input_shape: input_shape.clone(), output_shape: output_shape.clone() }
    }

    pub unsafe fn run(&self, stream: &HipStream, input: &DeviceTensor, output: &DeviceTensor) {
        assert_eq!(input.strided_shape(), &self.input_shape);
        assert_eq!(output.strided_shape(), &self.output_shape);
        self.raw.run(stream, &[input.ptr().ptr(), output.ptr().ptr()]);
    }
}

#[derive(Debug)]
pub struct SoftmaxKernel {
    raw: RawKernel,
    input_shape: StridedShape,
    output_shape: StridedShape,
}

impl SoftmaxKernel {
    pub fn new(device: HipDevice, input_shape: &StridedShape, output_shape: &StridedShape, softmax_axis: usize, input_scale: f32) -> Self {
        assert_eq!(input_shape.shape(), output_shape.shape());
        let (input, output) = (describe(input_shape, DType::F32), describe(output_shape, DType::F32));
        let mut raw = null_mut();
        unsafe { knhip_softmax_kernel_new(device.inner(), &input.raw, &output.raw, softmax_axis, input_scale, &mut raw) }.unwrap();
        SoftmaxKernel { raw: RawKernel(raw), input_shape: input_shape.clone(), output_shape: output_shape.clone() }
    }

    pub unsafe fn run(&self, stream: &HipStream, input: &DeviceTensor, output: &DeviceTensor) {
        assert_eq!(input.strided_shape(), &self.input_shape);
        assert_eq!(output.strided_shape(), &self.output_shape);
        self.raw.run(stream, &[input.ptr().ptr(), output.ptr().ptr()]);
    }
}

#[derive(Debug)]
pub struct LayernormKernel {
    raw: RawKernel,
    input_shape: StridedShape,
    output_shape: StridedShape,
    alpha1: f32,
}

impl LayernormKernel {
    #[allow(clippy::too_many_arguments)]
    pub fn new(device: HipDevice, input_shape: &StridedShape, output_shape: &StridedShape, norm_axis: usize, eps: f32, alpha_0: f32,
               alpha_1: f32, beta: f32) -> Self {
        assert_eq!(input_shape.shape(), output_shape.shape());
        let (input, output) = (describe(input_shape, DType::F32), describe(output_shape, DType::F32));
        let mut raw = null_mut();
        unsafe { knhip_layernorm_kernel_new(device.inner(), &input.raw, &output.raw, norm_axis, eps, alpha_0, alpha_1, beta, &mut raw) }
            .unwrap();
        LayernormKernel { raw: RawKernel(raw), input_shape: input_shape.clone(), output_shape: output_shape.clone(), alpha1: alpha_1 }
    }

    pub unsafe fn run(&self, stream: &HipStream, input0: &DeviceTensor, input1: Option<&DeviceTensor>, output: &DeviceTensor) {
        assert_eq!(input0.strided_shape(), &self.input_shape);
        if let Some(input1) = input1 {
            assert_eq!(input1.strided_shape(), &self.input_shape);
        }
        assert_eq!(output.strided_shape(), &self.output_shape);
        if self.alpha1 != 0.0 {
            assert!(input1.is_some());
        }
        let second = if self.alpha1 != 0.0 { input1.map_or(null_mut(), |x| x.ptr().ptr()) } else { null_mut() };
        self.raw.run(stream, &[input0.ptr().ptr(), second, output.ptr().ptr()]);
    }
}

#[derive(Debug)]
pub struct GatherKernel {
    raw: RawKernel,
    input_shape: StridedShape,
    indices_shape: StridedShape,
    output_shape: StridedShape,
    dtype: DType,
    itype: DType,
}

impl GatherKernel {
    pub fn new(device: HipDevice, input_shape: &StridedShape, indices_shape: &StridedShape, output_shape: &StridedShape, dtype: DType,
               itype: DType, axis: usize) -> Self {
        let (input, indices, output) = (describe(input_shape, dtype), describe(indices_shape, itype), describe(output_shape, dtype));
        let mut raw = null_mut();
        unsafe { knhip_gather_kernel_new(device.inner(), &input.raw, &indices.raw, &output.raw, axis, &mut raw) }.unwrap();
        GatherKernel {
            raw: RawKernel(raw),
            input_shape: input_shape.clone(),
            indices_shape: indices_shape.clone(),
            output_shape: output_shape.clone(),
            dtype,
            itype,
        }
    }

    pub unsafe fn run(&self, stream: &HipStream, input: &DeviceTensor, indices: &DeviceTensor, output: &DeviceTensor) {
        assert_eq!(input.strided_shape(), &self.input_shape);
        assert_eq!(indices.strided_shape(), &self.indices_shape);
        assert_eq!(output.strided_shape(), &self.output_shape);
        assert_eq!(input.dtype(), self.dtype);
        assert_eq!(indices.dtype(), self.itype);
        assert_eq!(output.dtype(), self.dtype);
        self.raw.run(stream, &[input.ptr().ptr(), indices.ptr().ptr(), output.ptr().ptr()]);
    }
}
