"""The run-time compiled kernel types of kn-cuda-eval/src/autokernel/ on caller-owned DeviceTensors: ScalarKernel
(scalar.rs:33-154), ReduceKernel (reduce.rs:35-153), SoftmaxKernel (softmax.rs:28-108), LayernormKernel
(layernorm.rs:33-136) and GatherKernel (gather.rs:30-129). Constructors take StridedShapes like the reference's; `run`
checks the tensors against them like the reference's asserts do. `device=None` compiles without a GPU."""
from ctypes import byref, c_int64, c_size_t, c_uint, c_void_p

from ._lib import KnError, TensorT, check, lib
from .device_tensor import StridedShape, _arr
from .graph import DType, ReduceOp
from .runtime import HipStream, _index


def _descriptor(shape, dtype, ptr=0):
    t = TensorT()
    t._shape, t._strides = _arr(c_size_t, shape.shape), _arr(c_int64, shape.strides)
    t.ptr, t.dtype, t.rank, t.shape, t.strides = ptr, int(DType(dtype)), shape.rank(), t._shape, t._strides
    return t


class _Kernel:
    def __init__(self, device, shapes, dtypes):
        self.device = -1 if device is None else _index(device)
        self.shapes, self.dtypes = list(shapes), [DType(d) for d in dtypes]
        self._h = c_void_p()

    def _run(self, stream, tensors):
        ptrs = []
        for i, (t, shape, dtype) in enumerate(zip(tensors, self.shapes, self.dtypes)):
            if t is None:
                ptrs.append(None)
                continue
            if t.strided_shape != shape:
                raise KnError(f"operand {i}: {t.strided_shape} does not match the kernel's {shape}")
            if t.dtype != dtype:
                raise KnError(f"operand {i}: dtype {t.dtype.name} does not match the kernel's {dtype.name}")
            ptrs.append(t.ptr)
        handle = stream._h if isinstance(stream, HipStream) else c_void_p(stream or 0)
        check(lib.knhip_kernel_run(self._h, handle, (c_void_p * max(len(ptrs), 1))(*ptrs), len(ptrs)))

    def info(self):
        """(strategy text, workgroups, threads per workgroup)"""
        needed, grid, block = c_size_t(), c_uint(), c_uint()
        check(lib.knhip_kernel_info(self._h, None, 0, byref(needed), byref(grid), byref(block)))
        import ctypes
        buf = ctypes.create_string_buffer(needed.value)
        check(lib.knhip_kernel_info(self._h, buf, needed.value, byref(needed), byref(grid), byref(block)))
        return buf.value.decode(), grid.value, block.value

    def __del__(self):
        if getattr(self, "_h", None) is not None and self._h.value and lib is not None:
            lib.knhip_kernel_free(self._h)
            self._h = None


class ScalarKernel(_Kernel):
    """`ScalarKernel.new_for_shapes(device, "*x0 = *x1 + *x2;", shapes, dtypes)`; operand 0 is written."""

    @staticmethod
    def new_for_shapes(device, operation, shapes, dtypes):
        if not shapes or len(shapes) != len(dtypes):
            raise KnError("one dtype per shape, and at least one operand")
        k = ScalarKernel(device, shapes, dtypes)
        descs = (TensorT * len(shapes))(*[_descriptor(s, d) for s, d in zip(shapes, dtypes)])
        k._keep = descs
        check(lib.knhip_scalar_kernel_new(k.device, operation.encode(), descs, len(shapes), byref(k._h)))
        return k

    def run(self, stream, tensors):
        if len(tensors) != len(self.shapes):
            raise KnError(f"expected {len(self.shapes)} tensors, got {len(tensors)}")
        self._run(stream, tensors)


class ReduceKernel(_Kernel):
    def __init__(self, device, op, input_shape, output_shape, reduced_axes, dtype=DType.F32):
        super().__init__(device, [input_shape, output_shape], [dtype, dtype])
        axes = _arr(c_size_t, list(reduced_axes))
        check(lib.knhip_reduce_kernel_new(self.device, int(ReduceOp(op)), byref(_descriptor(input_shape, dtype)),
                                          byref(_descriptor(output_shape, dtype)), axes, len(reduced_axes), byref(self._h)))

    def run(self, stream, input, output):
        self._run(stream, [input, output])


class SoftmaxKernel(_Kernel):
    def __init__(self, device, input_shape, output_shape, softmax_axis, input_scale=1.0):
        super().__init__(device, [input_shape, output_shape], [DType.F32, DType.F32])
        check(lib.knhip_softmax_kernel_new(self.device, byref(_descriptor(input_shape, DType.F32)),
                                           byref(_descriptor(output_shape, DType.F32)), softmax_axis, input_scale, byref(self._h)))

    def run(self, stream, input, output):
        self._run(stream, [input, output])


class LayernormKernel(_Kernel):
    def __init__(self, device, input_shape, output_shape, norm_axis, eps, alpha_0=1.0, alpha_1=0.0, beta=1.0):
        super().__init__(device, [input_shape, input_shape, output_shape], [DType.F32] * 3)
        self.alpha_1 = alpha_1
        check(lib.knhip_layernorm_kernel_new(self.device, byref(_descriptor(input_shape, DType.F32)),
                                             byref(_descriptor(output_shape, DType.F32)), norm_axis, eps, alpha_0, alpha_1, beta,
                                             byref(self._h)))

    def run(self, stream, input0, input1, output):
        if self.alpha_1 != 0.0 and input1 is None:
            raise KnError("input1 is needed when alpha_1 is not zero")  # layernorm.rs:109-111
        self._run(stream, [input0, input1 if self.alpha_1 != 0.0 else None, output])


class GatherKernel(_Kernel):
    def __init__(self, device, input_shape, indices_shape, output_shape, dtype, itype, axis):
        super().__init__(device, [input_shape, indices_shape, output_shape], [dtype, itype, dtype])
        check(lib.knhip_gather_kernel_new(self.device, byref(_descriptor(input_shape, dtype)), byref(_descriptor(indices_shape, itype)),
                                          byref(_descriptor(output_shape, dtype)), axis, byref(self._h)))

    def run(self, stream, input, indices, output):
        self._run(stream, [input, indices, output])
