"""DeviceTensor: a strided view of device memory that the caller owns, with the reference's methods
(kn-cuda-eval/src/device_tensor.rs:20-169 and the views of offset_tensor.rs:52-139), and StridedShape, the layout
algebra underneath (kn-cuda-eval/src/shape.rs:25-285), which the library computes (knhip_strided_*)."""
from ctypes import byref, c_int, c_int64, c_size_t, c_void_p

import numpy as np

from ._lib import KnError, TensorT, check, lib
from .graph import DType
from .runtime import DeviceBuffer, HipStream, _index


def _arr(ctype, values):
    return (ctype * max(len(values), 1))(*values)


class StridedShape:
    """shape + strides in elements (zero = broadcast, negative = flipped)"""

    def __init__(self, shape, strides):
        self.shape, self.strides = [int(d) for d in shape], [int(s) for s in strides]
        if len(self.shape) != len(self.strides):
            raise KnError(f"shape {self.shape} and strides {self.strides} differ in rank")

    @staticmethod
    def new_simple(shape):
        strides, run = [], 1
        for d in reversed(shape):
            strides.append(run)
            run *= int(d)
        return StridedShape(shape, strides[::-1])

    def rank(self):
        return len(self.shape)

    def size(self):
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def _flags(self):
        simple, dense = c_int(), c_int()
        check(lib.knhip_strided_flags(_arr(c_size_t, self.shape), _arr(c_int64, self.strides), self.rank(), byref(simple), byref(dense)))
        return bool(simple.value), bool(dense.value)

    def has_simple_strides(self):
        return self._flags()[0]

    def has_dense_strides(self):
        return self._flags()[1]

    def permute(self, permutation):
        if sorted(permutation) != list(range(self.rank())):
            raise KnError(f"invalid permutation {permutation} for rank {self.rank()}")
        return StridedShape([self.shape[p] for p in permutation], [self.strides[p] for p in permutation])

    def view(self, new_shape):
        """None when the view cannot be expressed as a stride edit (shape.rs:135-189)"""
        ok, out = c_int(), (c_int64 * max(len(new_shape), 1))()
        check(lib.knhip_strided_view(_arr(c_size_t, self.shape), _arr(c_int64, self.strides), self.rank(),
                                     _arr(c_size_t, list(new_shape)), len(new_shape), byref(ok), out))
        return StridedShape(new_shape, [out[i] for i in range(len(new_shape))]) if ok.value else None

    def broadcast(self, new_shape):
        if len(new_shape) < self.rank():
            raise KnError(f"cannot broadcast {self.shape} to {list(new_shape)}")
        pad = len(new_shape) - self.rank()
        strides = [0] * pad
        for d, s, n in zip(self.shape, self.strides, new_shape[pad:]):
            if d == n:
                strides.append(s)
            elif d == 1:
                strides.append(0)
            else:
                raise KnError(f"cannot broadcast {self.shape} to {list(new_shape)}")
        return StridedShape(new_shape, strides)

    def slice(self, axis, start, end, step=1):
        out_shape, out_strides = (c_size_t * max(self.rank(), 1))(), (c_int64 * max(self.rank(), 1))()
        check(lib.knhip_strided_slice(_arr(c_size_t, self.shape), _arr(c_int64, self.strides), self.rank(), axis, start, end, step,
                                      out_shape, out_strides))
        return StridedShape([out_shape[i] for i in range(self.rank())], [out_strides[i] for i in range(self.rank())])

    def flip(self, axis):
        strides = list(self.strides)
        strides[axis] = -strides[axis]
        return StridedShape(self.shape, strides)

    def repeat_unary(self, axis, count):
        if self.shape[axis] != 1:
            raise KnError(f"repeat_unary needs a unit axis, got {self.shape} axis {axis}")
        shape, strides = list(self.shape), list(self.strides)
        shape[axis], strides[axis] = count, 0
        return StridedShape(shape, strides)

    def __eq__(self, other):
        return isinstance(other, StridedShape) and self.shape == other.shape and self.strides == other.strides

    def __repr__(self):
        return f"StridedShape(shape={self.shape}, strides={self.strides})"


class DeviceTensor:
    """`PtrTensor<DevicePtr>`: an address inside a device buffer (kept alive by the tensor), a StridedShape and a dtype."""

    def __init__(self, buffer, ptr, shape, dtype):
        self.buffer, self.ptr, self.strided_shape, self.dtype = buffer, int(ptr), shape, DType(dtype)

    @staticmethod
    def from_parts(buffer, ptr, shape, dtype):
        return DeviceTensor(buffer, ptr, shape, dtype)

    @staticmethod
    def alloc_simple(device, shape, dtype=DType.F32):
        """device_tensor.rs:21-25"""
        dtype = DType(dtype)
        strided = StridedShape.new_simple(list(shape))
        buffer = DeviceBuffer(device, max(strided.size() * np.dtype(dtype.numpy).itemsize, 1))
        return DeviceTensor(buffer, buffer.ptr, strided, dtype)

    @property
    def device(self):
        return self.buffer.device

    def dense_size_bytes(self):
        return self.strided_shape.size() * np.dtype(self.dtype.numpy).itemsize

    def descriptor(self):
        """the `knhip_tensor` of this view; keeps its arrays alive as attributes"""
        t = TensorT()
        t._shape, t._strides = _arr(c_size_t, self.strided_shape.shape), _arr(c_int64, self.strided_shape.strides)
        t.ptr, t.dtype, t.rank = self.ptr, int(self.dtype), self.strided_shape.rank()
        t.shape, t.strides = t._shape, t._strides
        return t

    # ---- views (offset_tensor.rs:52-114): stride and address edits, nothing is copied
    def _offset(self, offset_elem, shape):
        return DeviceTensor(self.buffer, self.ptr + offset_elem * np.dtype(self.dtype.numpy).itemsize, shape, self.dtype)

    def permute(self, permutation):
        return self._offset(0, self.strided_shape.permute(permutation))

    def view(self, new_shape):
        shape = self.strided_shape.view(list(new_shape))
        if shape is None:
            raise KnError(f"cannot view {self.strided_shape} as {list(new_shape)} without a copy")
        return self._offset(0, shape)

    def broadcast(self, new_shape):
        return self._offset(0, self.strided_shape.broadcast(list(new_shape)))

    def slice(self, axis, start, end, step=1):
        result = self.strided_shape.slice(axis, start, end, step)
        offset = self.strided_shape.strides[axis] * start if result.size() != 0 else 0
        return self._offset(offset, result)

    def index(self, axis, index):
        shape = list(self.strided_shape.shape)
        del shape[axis]
        return self.slice(axis, index, index + 1).view(shape)

    def flip(self, axis):
        length = self.strided_shape.shape[axis]
        offset = (length - 1) * self.strided_shape.strides[axis] if self.strided_shape.size() != 0 and length != 0 else 0
        return self._offset(offset, self.strided_shape.flip(axis))

    def repeat_unary(self, axis, count):
        return self._offset(0, self.strided_shape.repeat_unary(axis, count))

    def to_mat_mul_arg(self):
        """(address, (batch, row, column) strides) for `matmul_args`, the role of offset_tensor.rs:118-139: rank 3,
        and like there one of the two matrix axes must be dense"""
        if self.strided_shape.rank() != 3:
            raise KnError("a matmul operand has rank 3")
        sb, sr, sc = self.strided_shape.strides
        if sr != 1 and sc != 1:
            raise KnError(f"GPU matmul operand must be either col- or row-dense, got {self.strided_shape}")
        return self.ptr, (sb, sr, sc)

    # ---- copies
    def copy_simple_from_host(self, array):
        """device_tensor.rs:38-52"""
        array = np.ascontiguousarray(array)
        if not self.strided_shape.has_simple_strides():
            raise KnError(f"Tensor must have simple strides, got {self.strided_shape}")
        if array.nbytes != self.dense_size_bytes() or array.dtype != self.dtype.numpy:
            raise KnError(f"Wrong buffer size {array.nbytes} or dtype {array.dtype} for {self.strided_shape} of {self.dtype.name}")
        if array.nbytes:
            check(lib.knhip_memcpy_h2d(self.device, c_void_p(self.ptr), array.ctypes.data, array.nbytes))

    def copy_simple_to_host(self):
        """device_tensor.rs:54-68; returns a new array"""
        if not self.strided_shape.has_simple_strides():
            raise KnError(f"Tensor must have simple strides, got {self.strided_shape}")
        out = np.empty(self.strided_shape.shape, self.dtype.numpy)
        if out.nbytes:
            check(lib.knhip_memcpy_d2h(self.device, out.ctypes.data, c_void_p(self.ptr), out.nbytes))
        return out

    def copy_from(self, other, stream=None):
        """device_tensor.rs:101-126: a linear copy when both sides have the same dense strides, else the elementwise
        kernel `y = x` on the two layouts. Like the reference it returns when the copy is done, unless a stream is given."""
        if self.device != other.device:
            raise KnError("Tensors must be on the same device")
        d, s = self.descriptor(), other.descriptor()
        handle = stream._h if isinstance(stream, HipStream) else c_void_p(stream or 0)
        check(lib.knhip_strided_copy(self.device, handle, byref(d), byref(s)))
        if stream is None:
            check(lib.knhip_stream_synchronize(self.device, handle))

    def deep_clone(self):
        """device_tensor.rs:31-36"""
        new = DeviceTensor.alloc_simple(self.device, self.strided_shape.shape, self.dtype)
        new.copy_from(self)
        return new

    def copy_from_host_staged(self, array):
        """device_tensor.rs:128-147 (there f32 only): any strides, through a dense stage on the device when needed"""
        if self.strided_shape.has_simple_strides():
            self.copy_simple_from_host(array)
            return
        stage = DeviceTensor.alloc_simple(self.device, self.strided_shape.shape, self.dtype)
        stage.copy_simple_from_host(array)
        self.copy_from(stage)

    def copy_to_host_staged(self):
        """device_tensor.rs:149-168"""
        if self.strided_shape.has_simple_strides():
            return self.copy_simple_to_host()
        stage = DeviceTensor.alloc_simple(self.device, self.strided_shape.shape, self.dtype)
        stage.copy_from(self)
        return stage.copy_simple_to_host()

    def __repr__(self):
        return f"DeviceTensor(ptr=0x{self.ptr:x}, {self.strided_shape}, {self.dtype.name})"
