//! Safe wrappers with the names and behaviour of `kn-cuda-sys/src/wrapper`: a failed call panics with the library's
//! message (status.rs:9-33), every call names its device (handle.rs:20-23), handles free themselves on drop.
use std::ffi::CStr;
use std::os::raw::{c_char, c_int, c_void};
use std::ptr::null_mut;
use std::sync::Arc;

use crate::*;

/// status.rs:18-23: any status other than success is a panic.
pub trait Status {
    fn unwrap(self);
    fn unwrap_in_drop(self);
}

pub fn last_error() -> String {
    unsafe { CStr::from_ptr(knhip_last_error()) }.to_string_lossy().into_owned()
}

impl Status for c_int {
    #[track_caller]
    fn unwrap(self) {
        if self != KNHIP_OK {
            panic!("knhip failure (status {}): {}", self, last_error());
        }
    }

    #[track_caller]
    fn unwrap_in_drop(self) {
        // status.rs:25-32: no second panic while unwinding
        if self != KNHIP_OK && !std::thread::panicking() {
            panic!("knhip failure (status {}): {}", self, last_error());
        }
    }
}

/// Reads a string through the (buf, cap, needed) protocol of the C ABI.
pub fn read_string(mut call: impl FnMut(*mut c_char, usize, *mut usize) -> c_int) -> String {
    let mut needed = 0usize;
    let status = call(null_mut(), 0, &mut needed);
    if status != KNHIP_OK && status != KNHIP_BUFFER_TOO_SMALL {
        status.unwrap();
    }
    let mut buf = vec![0u8; needed + 1];
    call(buf.as_mut_ptr() as *mut c_char, buf.len(), &mut needed).unwrap();
    let len = buf.iter().position(|&c| c == 0).unwrap_or(buf.len());
    String::from_utf8_lossy(&buf[..len]).into_owned()
}

/// A device index, the twin of `CudaDevice` (handle.rs:25-103).
#[derive(Debug, Copy, Clone, Eq, PartialEq, Hash)]
pub struct HipDevice(i32);

#[derive(Debug, Copy, Clone, Eq, PartialEq, Hash)]
pub struct HipDeviceNotAvailable;

fn hip_device_count() -> i32 {
    let mut count: c_int = 0;
    unsafe { knhip_device_count(&mut count) }.unwrap();
    count
}

impl HipDevice {
    pub fn new(device: i32) -> Result<Self, HipDeviceNotAvailable> {
        if 0 <= device && device < hip_device_count() {
            Ok(HipDevice(device))
        } else {
            Err(HipDeviceNotAvailable)
        }
    }

    pub fn all() -> impl Iterator<Item = Self> {
        (0..hip_device_count()).map(HipDevice)
    }

    pub fn inner(self) -> i32 {
        self.0
    }

    /// Nothing to do: every entry point of the library selects the device it is given. Kept so that code written
    /// against `CudaDevice::switch_to` ports by renaming.
    pub fn switch_to(self) {}

    pub fn alloc(self, len_bytes: usize) -> DevicePtr {
        DevicePtr::alloc(self, len_bytes)
    }

    pub fn name(self) -> String {
        read_string(|buf, cap, needed| unsafe { knhip_device_name(self.0, buf, cap, needed) })
    }

    pub fn synchronize(self) {
        unsafe { knhip_device_synchronize(self.0) }.unwrap()
    }
}

/// event.rs:7-45
#[derive(Debug)]
pub struct HipEvent {
    device: HipDevice,
    inner: *mut c_void,
}

impl HipEvent {
    pub fn new(device: HipDevice) -> Self {
        let mut inner = null_mut();
        unsafe { knhip_event_create(device.inner(), &mut inner) }.unwrap();
        HipEvent { device, inner }
    }

    /// Elapsed time since `start` in seconds.
    pub fn time_elapsed_since(&self, start: &HipEvent) -> f32 {
        let mut seconds = 0f32;
        unsafe { knhip_event_elapsed_seconds(self.device.inner(), start.inner, self.inner, &mut seconds) }.unwrap();
        seconds
    }

    pub fn synchronize(&self) {
        unsafe { knhip_event_synchronize(self.device.inner(), self.inner) }.unwrap()
    }

    pub unsafe fn inner(&self) -> *mut c_void {
        self.inner
    }
}

impl Drop for HipEvent {
    fn drop(&mut self) {
        unsafe { knhip_event_destroy(self.device.inner(), self.inner) }.unwrap_in_drop()
    }
}

/// handle.rs:105-174. A stream is owned, or borrowed from an executor (then it is not destroyed on drop).
#[derive(Debug)]
pub struct HipStream {
    device: HipDevice,
    inner: *mut c_void,
    owned: bool,
}

impl HipStream {
    pub fn new(device: HipDevice) -> Self {
        let mut inner = null_mut();
        unsafe { knhip_stream_create(device.inner(), &mut inner) }.unwrap();
        HipStream { device, inner, owned: true }
    }

    /// Safety: `inner` must be a live stream of `device` that outlives the returned value.
    pub unsafe fn borrowed(device: HipDevice, inner: *mut c_void) -> Self {
        HipStream { device, inner, owned: false }
    }

    pub fn synchronize(&self) {
        unsafe { knhip_stream_synchronize(self.device.inner(), self.inner) }.unwrap()
    }

    pub fn device(&self) -> HipDevice {
        self.device
    }

    pub unsafe fn inner(&self) -> *mut c_void {
        self.inner
    }

    pub fn record_event(&self) -> HipEvent {
        let event = HipEvent::new(self.device);
        self.record_existing_event(&event);
        event
    }

    pub fn record_existing_event(&self, event: &HipEvent) {
        unsafe { knhip_event_record(self.device.inner(), event.inner, self.inner) }.unwrap()
    }

    pub fn wait_for_event(&self, event: &HipEvent) {
        unsafe { knhip_stream_wait_event(self.device.inner(), self.inner, event.inner) }.unwrap()
    }
}

impl Drop for HipStream {
    fn drop(&mut self) {
        if self.owned {
            unsafe { knhip_stream_destroy(self.device.inner(), self.inner) }.unwrap_in_drop()
        }
    }
}

/// mem/pinned.rs
#[derive(Debug)]
pub struct PinnedMem {
    ptr: *mut c_void,
    len_bytes: usize,
}

impl PinnedMem {
    pub fn alloc(len_bytes: usize) -> Self {
        let mut ptr = null_mut();
        unsafe { knhip_host_alloc(len_bytes.max(1), &mut ptr) }.unwrap();
        PinnedMem { ptr, len_bytes }
    }

    pub unsafe fn ptr(&self) -> *mut c_void {
        self.ptr
    }

    pub fn len_bytes(&self) -> usize {
        self.len_bytes
    }

    /// Safety: no other slice exists and no device is writing to this memory.
    #[allow(clippy::mut_from_ref)]
    pub unsafe fn as_slice(&self) -> &mut [u8] {
        if self.len_bytes == 0 {
            &mut []
        } else {
            std::slice::from_raw_parts_mut(self.ptr as *mut u8, self.len_bytes)
        }
    }
}

impl Drop for PinnedMem {
    fn drop(&mut self) {
        unsafe { knhip_host_free(self.ptr) }.unwrap_in_drop()
    }
}

/// mem/device.rs:18-46: one allocation, freed when the last pointer into it is dropped. A buffer that somebody else
/// owns (the arena of an executor) is only described, never freed.
#[derive(Debug)]
struct DeviceBuffer {
    device: HipDevice,
    base: *mut c_void,
    len_bytes: usize,
    owned: bool,
}

unsafe impl Send for DeviceBuffer {}
unsafe impl Sync for DeviceBuffer {}

impl Drop for DeviceBuffer {
    fn drop(&mut self) {
        if self.owned {
            unsafe { knhip_free(self.device.inner(), self.base) }.unwrap_in_drop()
        }
    }
}

/// mem/device.rs:48-153: a reference counted allocation plus a byte offset into it.
#[derive(Debug, Clone)]
pub struct DevicePtr {
    buffer: Arc<DeviceBuffer>,
    offset_bytes: isize,
}

impl DevicePtr {
    pub fn alloc(device: HipDevice, len_bytes: usize) -> Self {
        let mut base = null_mut();
        unsafe { knhip_malloc(device.inner(), len_bytes.max(1), &mut base) }.unwrap();
        DevicePtr { buffer: Arc::new(DeviceBuffer { device, base, len_bytes, owned: true }), offset_bytes: 0 }
    }

    /// `len_bytes` of device memory at `base` that is owned elsewhere (an executor's input or output tensor).
    /// Safety: the memory outlives every pointer made from the result.
    pub unsafe fn borrowed(device: HipDevice, base: *mut c_void, len_bytes: usize) -> Self {
        DevicePtr { buffer: Arc::new(DeviceBuffer { device, base, len_bytes, owned: false }), offset_bytes: 0 }
    }

    pub fn device(&self) -> HipDevice {
        self.buffer.device
    }

    pub fn offset_bytes(self, offset: isize) -> DevicePtr {
        let new_offset = self.offset_bytes + offset;
        assert!(0 <= new_offset && new_offset as usize <= self.buffer.len_bytes, "offset {} leaves the buffer", new_offset);
        DevicePtr { buffer: self.buffer, offset_bytes: new_offset }
    }

    pub unsafe fn ptr(&self) -> *mut c_void {
        (self.buffer.base as *mut u8).offset(self.offset_bytes) as *mut c_void
    }

    fn room(&self) -> usize {
        self.buffer.len_bytes - self.offset_bytes as usize
    }

    pub unsafe fn copy_linear_from_host(&self, buffer: &[u8]) {
        assert!(buffer.len() <= self.room());
        knhip_memcpy_h2d(self.device().inner(), self.ptr(), buffer.as_ptr() as *const c_void, buffer.len()).unwrap()
    }

    pub unsafe fn copy_linear_to_host(&self, buffer: &mut [u8]) {
        assert!(buffer.len() <= self.room());
        knhip_memcpy_d2h(self.device().inner(), buffer.as_mut_ptr() as *mut c_void, self.ptr(), buffer.len()).unwrap()
    }

    pub unsafe fn copy_linear_from_device(&self, other: &DevicePtr, len_bytes: usize) {
        assert_eq!(self.device(), other.device());
        assert!(len_bytes <= self.room() && len_bytes <= other.room());
        knhip_memcpy_d2d(self.device().inner(), self.ptr(), other.ptr(), len_bytes).unwrap()
    }

    /// mem/device.rs:114-132. The pinned memory must stay untouched until `stream` has passed the copy.
    pub unsafe fn copy_linear_from_host_async(&self, buffer: &PinnedMem, len_bytes: usize, stream: &HipStream) {
        assert!(len_bytes <= self.room() && len_bytes <= buffer.len_bytes());
        knhip_memcpy_h2d_async(self.device().inner(), self.ptr(), buffer.ptr(), len_bytes, stream.inner()).unwrap()
    }

    /// mem/device.rs:134-153
    pub unsafe fn copy_linear_to_host_async(&self, buffer: &PinnedMem, len_bytes: usize, stream: &HipStream) {
        assert!(len_bytes <= self.room() && len_bytes <= buffer.len_bytes());
        knhip_memcpy_d2h_async(self.device().inner(), buffer.ptr(), self.ptr(), len_bytes, stream.inner()).unwrap()
    }
}

/// `knhip_executor_options` with the library's defaults; change fields before building an executor. The options
/// belong to that executor alone: nothing is read from the environment.
#[derive(Debug, Copy, Clone)]
pub struct ExecutorOptions(pub knhip_executor_options);

impl Default for ExecutorOptions {
    fn default() -> Self {
        let mut raw = std::mem::MaybeUninit::<knhip_executor_options>::zeroed();
        unsafe {
            knhip_executor_options_default(raw.as_mut_ptr()).unwrap();
            ExecutorOptions(raw.assume_init())
        }
    }
}

impl ExecutorOptions {
    /// for callers that write the device inputs once and call `run_async` many times
    pub fn preserve_inputs(mut self) -> Self {
        self.0.preserve_inputs = 1;
        self
    }
}

/// Resolves the address of the static scratch of `knhip_batched_mat_mul_static` on `device`; call it once before a
/// stream capture that will contain `run_static`.
pub fn static_scratch_prepare(device: HipDevice) {
    unsafe { knhip_static_scratch_prepare(device.inner()) }.unwrap()
}

/// One matrix of a batched product: group.rs:87-105 (`MatMulOperand`), with element strides spelled out
/// instead of (transpose flag, leading dimension).
#[derive(Debug, Clone)]
pub struct MatMulOperand {
    pub ptr: DevicePtr,
    pub batch_stride: i64,
    pub row_stride: i64,
    pub col_stride: i64,
}

/// group.rs:107-171: `C[b] = A[b] B[b]`, f32 or f16 (code `KNHIP_F32` / `KNHIP_F16`).
#[derive(Debug, Clone)]
pub struct BatchedMatMulArgs {
    pub dtype: c_int,
    pub batch: usize,
    pub m: usize,
    pub n: usize,
    pub k: usize,
    pub a: MatMulOperand,
    pub b: MatMulOperand,
    pub c: MatMulOperand,
}

impl BatchedMatMulArgs {
    fn raw(&self) -> knhip_matmul_args {
        unsafe {
            knhip_matmul_args {
                dtype: self.dtype,
                batch: self.batch as c_int,
                m: self.m as c_int,
                n: self.n as c_int,
                k: self.k as c_int,
                a: self.a.ptr.ptr(),
                a_batch_stride: self.a.batch_stride,
                a_row_stride: self.a.row_stride,
                a_col_stride: self.a.col_stride,
                b: self.b.ptr.ptr(),
                b_batch_stride: self.b.batch_stride,
                b_row_stride: self.b.row_stride,
                b_col_stride: self.b.col_stride,
                c: self.c.ptr.ptr(),
                c_batch_stride: self.c.batch_stride,
                c_row_stride: self.c.row_stride,
                c_col_stride: self.c.col_stride,
            }
        }
    }

    pub fn workspace_bytes(&self) -> usize {
        let mut bytes = 0usize;
        unsafe { knhip_batched_mat_mul_workspace_bytes(&self.raw(), &mut bytes) }.unwrap();
        bytes
    }

    /// Queues the product on `stream`. `workspace` holds at least `workspace_bytes()` bytes (None when that is 0)
    /// and stays untouched until the work has run.
    pub unsafe fn run(&self, stream: &HipStream, workspace: Option<(&DevicePtr, usize)>) {
        let (ws, ws_bytes) = match workspace {
            Some((ptr, bytes)) => (ptr.ptr(), bytes),
            None => (null_mut(), 0),
        };
        knhip_batched_mat_mul(stream.device().inner(), stream.inner(), &self.raw(), ws, ws_bytes).unwrap()
    }

    /// The variant that allocates nothing: scratch comes from a static device array of
    /// `KNHIP_STATIC_SCRATCH_BYTES` per GPU, shared by all calls on that GPU (overlapping calls race).
    pub unsafe fn run_static(&self, stream: &HipStream) {
        knhip_batched_mat_mul_static(stream.device().inner(), stream.inner(), &self.raw()).unwrap()
    }
}
