//! `kn-hip-eval`: the GPU executor of Kyanite on AMD MI355X. Same surface as `kn-cuda-eval`
//! (`CudaExecutor::new / evaluate / run_async`, executor.rs:61, :117, :199); planning, kernel generation and
//! execution happen behind the C ABI of libknhip, this crate serialises the graph and moves tensors.
pub mod autokernel;
pub mod device_tensor;
pub mod executor;
pub mod serialize;
pub mod shape;

pub use kn_hip_sys::wrapper::{ExecutorOptions, HipDevice};

pub use crate::device_tensor::DeviceTensor;
pub use crate::executor::{HipExecutor, MemoryUsage, Profile};
