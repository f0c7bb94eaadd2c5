"""Streams, events, device and pinned memory and the stand-alone batched matrix product: the ctypes face of the
runtime tier of the C ABI, shaped like kn-cuda-sys's wrappers (CudaStream handle.rs:105-174, CudaEvent event.rs,
DevicePtr mem/device.rs, PinnedMem mem/pinned.rs, BatchedMatMulArgs group.rs:107-171)."""
import ctypes
from ctypes import byref, c_float, c_size_t, c_void_p

import numpy as np

from ._lib import KnError, MatmulArgsT, check, lib
from .graph import DType


def _index(device):
    return device.index if hasattr(device, "index") else int(device)


class HipEvent:
    def __init__(self, device=0):
        self.device = _index(device)
        h = c_void_p()
        check(lib.knhip_event_create(self.device, byref(h)))
        self._h = h

    def synchronize(self):
        check(lib.knhip_event_synchronize(self.device, self._h))

    def time_elapsed_since(self, start):
        """seconds, like CudaEvent::time_elapsed_since"""
        s = c_float()
        check(lib.knhip_event_elapsed_seconds(self.device, start._h, self._h, byref(s)))
        return s.value

    def __del__(self):
        if getattr(self, "_h", None) is not None and lib is not None:
            lib.knhip_event_destroy(self.device, self._h)
            self._h = None


class HipStream:
    """An owned stream, or a borrowed one (`HipStream.borrowed(device, handle)`, e.g. an executor's)."""

    def __init__(self, device=0):
        self.device = _index(device)
        h = c_void_p()
        check(lib.knhip_stream_create(self.device, byref(h)))
        self._h, self._owned = h, True

    @staticmethod
    def borrowed(device, handle):
        s = HipStream.__new__(HipStream)
        s.device, s._h, s._owned = _index(device), c_void_p(handle), False
        return s

    @property
    def handle(self):
        return self._h.value or 0

    def synchronize(self):
        check(lib.knhip_stream_synchronize(self.device, self._h))

    def record_event(self):
        event = HipEvent(self.device)
        self.record_existing_event(event)
        return event

    def record_existing_event(self, event):
        check(lib.knhip_event_record(self.device, event._h, self._h))

    def wait_for_event(self, event):
        check(lib.knhip_stream_wait_event(self.device, self._h, event._h))

    def __del__(self):
        if getattr(self, "_owned", False) and self._h is not None and lib is not None:
            lib.knhip_stream_destroy(self.device, self._h)
            self._h = None


class PinnedMem:
    """Page-locked host memory, seen as a numpy array through `array(dtype, shape)`."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = c_void_p()
        check(lib.knhip_host_alloc(self.nbytes, byref(p)))
        self.ptr = p.value

    def array(self, dtype, shape):
        count = int(np.prod(shape)) if len(shape) else 1
        assert count * np.dtype(dtype).itemsize <= self.nbytes
        buf = (ctypes.c_uint8 * self.nbytes).from_address(self.ptr)
        return np.frombuffer(buf, dtype=dtype, count=count).reshape(shape)

    def __del__(self):
        if getattr(self, "ptr", None) and lib is not None:
            lib.knhip_host_free(c_void_p(self.ptr))
            self.ptr = None


class DeviceBuffer:
    """Owned device memory (DevicePtr::alloc) with synchronous and stream-ordered copies."""

    def __init__(self, device, nbytes):
        self.device, self.nbytes = _index(device), int(nbytes)
        p = c_void_p()
        check(lib.knhip_malloc(self.device, self.nbytes, byref(p)))
        self.ptr = p.value

    @staticmethod
    def from_array(device, array):
        array = np.ascontiguousarray(array)
        buf = DeviceBuffer(device, max(array.nbytes, 1))
        if array.nbytes:
            check(lib.knhip_memcpy_h2d(buf.device, c_void_p(buf.ptr), array.ctypes.data, array.nbytes))
        return buf

    def to_array(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(lib.knhip_memcpy_d2h(self.device, out.ctypes.data, c_void_p(self.ptr), out.nbytes))
        return out

    def copy_from_host_async(self, pinned, nbytes, stream, offset=0):
        check(lib.knhip_memcpy_h2d_async(self.device, c_void_p(self.ptr + offset), c_void_p(pinned.ptr), nbytes, stream._h))

    def copy_to_host_async(self, pinned, nbytes, stream, offset=0):
        check(lib.knhip_memcpy_d2h_async(self.device, c_void_p(pinned.ptr), c_void_p(self.ptr + offset), nbytes, stream._h))

    def __del__(self):
        if getattr(self, "ptr", None) and lib is not None:
            lib.knhip_free(self.device, c_void_p(self.ptr))
            self.ptr = None


def matmul_args(dtype, batch, m, n, k, a, a_strides, b, b_strides, c, c_strides):
    """`a`, `b`, `c`: device addresses; strides: (batch, row, column) in elements."""
    args = MatmulArgsT()
    args.dtype, args.batch, args.m, args.n, args.k = int(DType(dtype)), batch, m, n, k
    args.a, (args.a_batch_stride, args.a_row_stride, args.a_col_stride) = a, a_strides
    args.b, (args.b_batch_stride, args.b_row_stride, args.b_col_stride) = b, b_strides
    args.c, (args.c_batch_stride, args.c_row_stride, args.c_col_stride) = c, c_strides
    return args


def batched_mat_mul_workspace_bytes(args):
    n = c_size_t()
    check(lib.knhip_batched_mat_mul_workspace_bytes(byref(args), byref(n)))
    return n.value


def batched_mat_mul(device, stream, args, workspace=None):
    """Queue C = A B on `stream`; `workspace` is a DeviceBuffer of at least `batched_mat_mul_workspace_bytes(args)`."""
    handle = stream._h if isinstance(stream, HipStream) else c_void_p(stream)
    ptr, size = (c_void_p(workspace.ptr), workspace.nbytes) if workspace is not None else (None, 0)
    check(lib.knhip_batched_mat_mul(_index(device), handle, byref(args), ptr, size))


STATIC_SCRATCH_BYTES = 32 << 20


def batched_mat_mul_static(device, stream, args):
    """`batched_mat_mul` on the library's static scratch (at most STATIC_SCRATCH_BYTES): allocates nothing."""
    handle = stream._h if isinstance(stream, HipStream) else c_void_p(stream)
    check(lib.knhip_batched_mat_mul_static(_index(device), handle, byref(args)))
