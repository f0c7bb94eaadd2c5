"""kyanite_amd: an MI355X (gfx950) executor for Kyanite graphs.

The work is done by libknhip.so (C++ host runtime + HIP kernels); this package is the ctypes face of its C ABI,
shaped like the reference's `kn-graph` builder and `CudaExecutor`.
"""
from ._lib import KnError, LIB_PATH
from .executor import Device, HipDevice, HipExecutor, PreparedGraph, Profile, compile_stats
from .runtime import (STATIC_SCRATCH_BYTES, DeviceBuffer, HipEvent, HipStream, PinnedMem, batched_mat_mul,
                      batched_mat_mul_static, batched_mat_mul_workspace_bytes, matmul_args)
from .device_tensor import DeviceTensor, StridedShape
from .autokernel import GatherKernel, LayernormKernel, ReduceKernel, ScalarKernel, SoftmaxKernel
from .graph import (BATCH, BINARY_ALL, REDUCE_ALL, UNARY_ALL, BinaryOp, DType, Graph, OpKind, OptimizerSettings,
                    ReduceOp, Size, UnaryOp, Value, optimize_graph, shape)

__all__ = [
    "KnError", "LIB_PATH", "Device", "HipDevice", "HipExecutor", "PreparedGraph", "Profile", "compile_stats",
    "BATCH", "BINARY_ALL", "REDUCE_ALL", "UNARY_ALL", "BinaryOp", "DType", "Graph", "OpKind", "OptimizerSettings",
    "ReduceOp", "Size", "UnaryOp", "Value", "optimize_graph", "shape",
    "DeviceBuffer", "HipEvent", "HipStream", "PinnedMem", "batched_mat_mul", "batched_mat_mul_workspace_bytes", "matmul_args",
    "STATIC_SCRATCH_BYTES", "batched_mat_mul_static",
    "DeviceTensor", "StridedShape", "ScalarKernel", "ReduceKernel", "SoftmaxKernel", "LayernormKernel", "GatherKernel",
]
