//! `DeviceTensor`: a strided view of device memory, with the methods of kn-cuda-eval/src/device_tensor.rs:20-169 and the
//! views of kn-cuda-eval/src/offset_tensor.rs:52-139. Copies between different layouts run the library's elementwise
//! kernel with the operation `y = x` (`knhip_strided_copy`).
use std::os::raw::c_void;
use std::ptr::null_mut;

use kn_graph::dtype::DType;
use kn_graph::graph::SliceRange;
use kn_hip_sys::wrapper::{DevicePtr, HipDevice, HipStream, MatMulOperand, Status};
use kn_hip_sys::{knhip_strided_copy, knhip_tensor};

use crate::serialize::dtype_code;
use crate::shape::{StridedShape, ViewError};

#[derive(Debug, Clone)]
pub struct DeviceTensor {
    ptr: DevicePtr,
    dtype: DType,
    shape: StridedShape,
}

/// The `knhip_tensor` of a tensor together with the arrays it points into.
pub struct TensorDescriptor {
    pub raw: knhip_tensor,
    _shape: Vec<usize>,
    _strides: Vec<i64>,
}

impl DeviceTensor {
    pub fn from_parts(ptr: DevicePtr, shape: StridedShape, dtype: DType) -> Self {
        DeviceTensor { ptr, dtype, shape }
    }

    pub fn alloc_simple(device: HipDevice, shape: Vec<usize>, dtype: DType) -> Self {
        let shape = StridedShape::new_simple(shape);
        let ptr = DevicePtr::alloc(device, shape.size() * dtype.size().bytes());
        DeviceTensor::from_parts(ptr, shape, dtype)
    }

    pub fn ptr(&self) -> &DevicePtr {
        &self.ptr
    }

    pub fn strided_shape(&self) -> &StridedShape {
        &self.shape
    }

    pub fn dtype(&self) -> DType {
        self.dtype
    }

    pub fn device(&self) -> HipDevice {
        self.ptr.device()
    }

    pub fn dense_size_bytes(&self) -> usize {
        self.shape.size() * self.dtype.size().bytes()
    }

    /// Safety: the descriptor holds a raw device address; the tensor must outlive its use.
    pub unsafe fn descriptor(&self) -> TensorDescriptor {
        let shape = self.shape.shape().to_vec();
        let strides = self.shape.strides_i64();
        let raw = knhip_tensor {
            ptr: self.ptr.ptr(),
            dtype: dtype_code(self.dtype) as std::os::raw::c_int,
            rank: shape.len(),
            shape: shape.as_ptr(),
            strides: strides.as_ptr(),
        };
        TensorDescriptor { raw, _shape: shape, _strides: strides }
    }

    // ---- views: stride and address edits, nothing is copied (offset_tensor.rs:52-114)
    fn offset(&self, offset_elem: isize, shape: StridedShape) -> Self {
        let offset_bytes = self.dtype.size().bytes() as isize * offset_elem;
        DeviceTensor::from_parts(self.ptr.clone().offset_bytes(offset_bytes), shape, self.dtype)
    }

    pub fn permute(&self, permutation: &[usize]) -> Self {
        self.offset(0, self.shape.permute(permutation))
    }

    pub fn view(&self, new_shape: Vec<usize>) -> Result<Self, ViewError> {
        self.shape.view(new_shape).map(|shape| self.offset(0, shape))
    }

    pub fn broadcast(&self, new_shape: Vec<usize>) -> Self {
        self.offset(0, self.shape.broadcast(new_shape))
    }

    pub fn slice(&self, axis: usize, range: impl Into<SliceRange>) -> Self {
        let range = range.into();
        let result_shape = self.shape.slice(axis, range);
        let offset = if result_shape.size() != 0 { self.shape.strides()[axis] * range.start as isize } else { 0 };
        self.offset(offset, result_shape)
    }

    pub fn index(&self, axis: usize, index: usize) -> Self {
        let mut new_shape = self.shape.shape().to_vec();
        new_shape.remove(axis);
        self.slice(axis, SliceRange::simple(index, index + 1)).view(new_shape).unwrap()
    }

    pub fn flip(&self, axis: usize) -> Self {
        let axis_len = self.shape.shape()[axis];
        let offset = if self.shape.size() != 0 && axis_len != 0 { (axis_len - 1) as isize * self.shape.strides()[axis] } else { 0 };
        self.offset(offset, self.shape.flip(axis))
    }

    pub fn repeat_unary(&self, axis: usize, count: usize) -> Self {
        self.offset(0, self.shape.repeat_unary(axis, count))
    }

    /// offset_tensor.rs:118-139, with element strides where cuBLAS wants a transpose flag and a leading dimension.
    pub fn to_mat_mul_arg(&self) -> MatMulOperand {
        assert_eq!(self.shape.rank(), 3);
        let s = self.shape.strides();
        assert!(s[1] == 1 || s[2] == 1, "GPU matmul operand must be either col- or row-dense, got {:?}", self.shape);
        MatMulOperand { ptr: self.ptr.clone(), batch_stride: s[0] as i64, row_stride: s[1] as i64, col_stride: s[2] as i64 }
    }

    // ---- copies
    pub fn deep_clone(&self) -> DeviceTensor {
        let new = DeviceTensor::alloc_simple(self.device(), self.shape.shape().to_vec(), self.dtype);
        unsafe { new.copy_from(self) };
        new
    }

    pub unsafe fn copy_simple_from_host(&self, buffer: &[u8]) {
        assert!(self.shape.has_simple_strides(), "Tensor must have simple strides, got {:?}", self);
        assert_eq!(buffer.len(), self.dense_size_bytes(), "Wrong buffer size {} for {:?}", buffer.len(), self);
        self.ptr.copy_linear_from_host(buffer);
    }

    pub unsafe fn copy_simple_to_host(&self, buffer: &mut [u8]) {
        assert!(self.shape.has_simple_strides(), "Tensor must have simple strides, got {:?}", self);
        assert_eq!(self.dense_size_bytes(), buffer.len(), "Wrong buffer size {} for {:?}", buffer.len(), self);
        self.ptr.copy_linear_to_host(buffer);
    }

    /// Queues `self[i] = other[i]` on `stream` (a null stream pointer is the device's default stream).
    pub unsafe fn copy_from_async(&self, other: &DeviceTensor, stream: *mut c_void) {
        assert_eq!(self.dtype, other.dtype, "Tensors must have the same dtype");
        assert_eq!(self.device(), other.device(), "Tensors must be on the same device");
        assert_eq!(self.shape.shape(), other.shape.shape(), "Tensors must have the same shape: {:?} vs {:?}", self, other);
        let (dst, src) = (self.descriptor(), other.descriptor());
        knhip_strided_copy(self.device().inner(), stream, &dst.raw, &src.raw).unwrap();
    }

    /// device_tensor.rs:101-126: done when it returns, like there.
    pub unsafe fn copy_from(&self, other: &DeviceTensor) {
        let stream = HipStream::new(self.device());
        self.copy_from_async(other, stream.inner());
        stream.synchronize();
    }

    /// device_tensor.rs:128-147 (any dtype here)
    pub unsafe fn copy_from_host_staged(&self, buffer: &[u8]) {
        assert_eq!(self.dense_size_bytes(), buffer.len(), "Wrong buffer size for {:?}", self.shape);
        if self.shape.has_simple_strides() {
            self.copy_simple_from_host(buffer);
        } else {
            let stage = DeviceTensor::alloc_simple(self.device(), self.shape.shape().to_vec(), self.dtype);
            stage.copy_simple_from_host(buffer);
            self.copy_from(&stage);
        }
    }

    /// device_tensor.rs:149-168
    pub unsafe fn copy_to_host_staged(&self, buffer: &mut [u8]) {
        assert_eq!(self.dense_size_bytes(), buffer.len(), "Wrong buffer size for {:?}", self.shape);
        if self.shape.has_simple_strides() {
            self.copy_simple_to_host(buffer);
        } else {
            let stage = DeviceTensor::alloc_simple(self.device(), self.shape.shape().to_vec(), self.dtype);
            stage.copy_from(self);
            stage.copy_simple_to_host(buffer);
        }
    }
}

/// `knhip_tensor` of an optional tensor for kernels that take one (a null pointer otherwise).
pub(crate) fn raw_or_null(descriptor: Option<&TensorDescriptor>) -> *const knhip_tensor {
    descriptor.map_or(null_mut() as *const knhip_tensor, |d| &d.raw as *const knhip_tensor)
}
