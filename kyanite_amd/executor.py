"""HipExecutor and the runtime device selector, mirroring kn-cuda-eval's CudaExecutor
(executor.rs:60-266) and kn-runtime's Device / PreparedGraph (kn-runtime/src/lib.rs:68-126)."""
import ctypes
from ctypes import byref, c_double, c_float, c_int, c_size_t, c_void_p

import numpy as np

from ._lib import ExecutorOptionsT, KnError, MemUsageT, ProfileT, check, get_string, lib
from .graph import DType, Graph

STEP_KINDS = ["conv", "mat_mul", "scalar_op", "reduce_op", "softmax_op", "layernorm_op", "gather_op"]


class HipDevice:
    """kn-cuda-sys/src/wrapper/handle.rs:37-103"""

    def __init__(self, index=0):
        n = HipDevice.count()
        if not 0 <= index < n:
            raise KnError(f"HIP device {index} is not available ({n} device(s) visible)")
        self.index = index

    @staticmethod
    def count():
        n = c_int()
        check(lib.knhip_device_count(byref(n)))
        return n.value

    @staticmethod
    def all():
        return [HipDevice(i) for i in range(HipDevice.count())]

    def name(self):
        return get_string(lib.knhip_device_name, self.index)

    def __repr__(self):
        return f"HipDevice({self.index})"


class Profile:
    def __init__(self, raw, step_seconds, text):
        for i, k in enumerate(STEP_KINDS):
            setattr(self, k, raw.per_kind[i])
        self.total_cpu = raw.total_cpu
        self.total_gpu = raw.total_gpu
        self.timing_overhead = raw.timing_overhead
        self.step_seconds = step_seconds
        self.text = text

    def __str__(self):
        return self.text


def executor_options(**fields):
    """A `knhip_executor_options` struct with the library's defaults and the given fields changed."""
    opts = ExecutorOptionsT()
    check(lib.knhip_executor_options_default(byref(opts)))
    known = {name for name, _ in ExecutorOptionsT._fields_} - {"struct_bytes"}
    for name, value in fields.items():
        if name not in known:
            raise KnError(f"unknown executor option {name!r}; known: {sorted(known)}")
        setattr(opts, name, int(value))
    return opts


class HipExecutor:
    """`HipExecutor(device, graph, batch_size)` / `evaluate(inputs) -> outputs`."""

    def __init__(self, device, graph, batch_size, plan_only=False, preserve_inputs=False, step_by_step=False, **options):
        """`options`: any further field of `knhip_executor_options` (include/knhip.h), e.g. `fuse_attention=False`,
        `mapped_io_bytes=0`; what is not named keeps its default. The options belong to this executor alone."""
        index = device.index if isinstance(device, HipDevice) else int(device)
        h = c_void_p()
        opts = executor_options(plan_only=plan_only, preserve_inputs=preserve_inputs, step_by_step=step_by_step, **options)
        check(lib.knhip_executor_new(index, graph._h, batch_size, byref(opts), byref(h)))
        self._h = h
        self.device = index
        self.batch_size = batch_size
        self.plan_only = plan_only
        n_in, n_out = c_size_t(), c_size_t()
        check(lib.knhip_executor_io_count(h, byref(n_in), byref(n_out)))
        self.input_info = [self._io_info(0, i) for i in range(n_in.value)]
        self.output_info = [self._io_info(1, i) for i in range(n_out.value)]

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and lib is not None:
            lib.knhip_executor_free(h)
            self._h = None

    def _io_info(self, is_output, i):
        dtype, rank = c_int(), c_size_t()
        check(lib.knhip_executor_io_info(self._h, is_output, i, byref(dtype), byref(rank), None, 0))
        dims = (c_size_t * max(rank.value, 1))()
        check(lib.knhip_executor_io_info(self._h, is_output, i, byref(dtype), byref(rank), dims, rank.value))
        return DType(dtype.value), [dims[k] for k in range(rank.value)]

    def evaluate(self, inputs, out=None):
        """Dense numpy arrays in, numpy arrays out: freshly allocated ones, or the dense arrays of `out` (as the
        reference hands out the same tensors again on every call, executor.rs:117, 194). Shapes and dtypes are checked
        like executor.rs:118-127 does."""
        if len(inputs) != len(self.input_info):
            raise KnError(f"Wrong input count: expected {len(self.input_info)}, got {len(inputs)}")
        arrays = []
        for i, (x, (dtype, dims)) in enumerate(zip(inputs, self.input_info)):
            x = np.asarray(x)
            if list(x.shape) != dims:
                raise KnError(f"Wrong shape for input {i}: expected {dims}, got {list(x.shape)}")
            if x.dtype != dtype.numpy:
                raise KnError(f"Wrong dtype for input {i}: expected {dtype.name}, got {x.dtype}")
            arrays.append(np.ascontiguousarray(x))
        if out is None:
            outputs = [np.empty(dims, dtype.numpy) for dtype, dims in self.output_info]
        else:
            outputs = list(out)
            if len(outputs) != len(self.output_info):
                raise KnError(f"Wrong output count: expected {len(self.output_info)}, got {len(outputs)}")
            for i, (y, (dtype, dims)) in enumerate(zip(outputs, self.output_info)):
                if not isinstance(y, np.ndarray) or list(y.shape) != dims or y.dtype != dtype.numpy or not y.flags.c_contiguous \
                        or not y.flags.writeable:
                    raise KnError(f"Output {i} must be a writeable dense {dtype.name} array of shape {dims}")
        n_in, n_out = len(arrays), len(outputs)
        in_ptrs = (c_void_p * max(n_in, 1))(*[a.ctypes.data for a in arrays])
        in_bytes = (c_size_t * max(n_in, 1))(*[a.nbytes for a in arrays])
        out_ptrs = (c_void_p * max(n_out, 1))(*[a.ctypes.data for a in outputs])
        out_bytes = (c_size_t * max(n_out, 1))(*[a.nbytes for a in outputs])
        check(lib.knhip_executor_evaluate(self._h, in_ptrs, in_bytes, n_in, out_ptrs, out_bytes, n_out))
        return outputs

    def run_async(self):
        check(lib.knhip_executor_run_async(self._h))

    def synchronize(self):
        check(lib.knhip_executor_synchronize(self._h))

    def time_runs(self, iterations):
        """Device milliseconds for `iterations` back-to-back runs (events on the executor's stream)."""
        ms = c_float()
        check(lib.knhip_executor_time_runs(self._h, iterations, byref(ms)))
        return ms.value

    def upload_input(self, i, array):
        """Copy a host array into input `i` on the device (for callers that drive `run_async` themselves)."""
        dtype, dims = self.input_info[i]
        array = np.ascontiguousarray(array)
        if list(array.shape) != dims or array.dtype != dtype.numpy:
            raise KnError(f"Wrong shape or dtype for input {i}")
        if array.nbytes:
            check(lib.knhip_memcpy_h2d(self.device, self.input_ptr(i), array.ctypes.data, array.nbytes))

    def download_output(self, i, rows=None):
        """Copy output `i` (or its first `rows` entries along axis 0) back to the host."""
        dtype, dims = self.output_info[i]
        if rows is not None:
            dims = [min(rows, dims[0])] + dims[1:]
        out = np.empty(dims, dtype.numpy)
        if out.nbytes:
            check(lib.knhip_memcpy_d2h(self.device, out.ctypes.data, self.output_ptr(i), out.nbytes))
        return out

    def input_ptr(self, i):
        p = c_void_p()
        check(lib.knhip_executor_input_ptr(self._h, i, byref(p)))
        return p.value

    def output_ptr(self, i):
        p = c_void_p()
        check(lib.knhip_executor_output_ptr(self._h, i, byref(p)))
        return p.value

    def stream(self):
        p = c_void_p()
        check(lib.knhip_executor_stream(self._h, byref(p)))
        return p.value or 0

    def set_graph_mode(self, enabled):
        """Replay the launch list as one HIP graph (captured on the first run) instead of launching every step."""
        check(lib.knhip_executor_set_graph_mode(self._h, int(enabled)))

    def set_profile(self, enabled):
        check(lib.knhip_executor_set_profile(self._h, int(enabled)))

    def last_profile(self):
        available, raw = c_int(), ProfileT()
        check(lib.knhip_executor_last_profile(self._h, byref(available), byref(raw)))
        if not available.value:
            return None
        buf = (c_float * max(raw.step_count, 1))()
        check(lib.knhip_executor_profile_step_seconds(self._h, buf, raw.step_count))
        text = get_string(lib.knhip_executor_profile_str, self._h)
        return Profile(raw, [buf[i] for i in range(raw.step_count)], text)

    @property
    def mem_usage(self):
        u = MemUsageT()
        check(lib.knhip_executor_mem_usage(self._h, byref(u)))
        return {name: getattr(u, name) for name, _ in MemUsageT._fields_}

    def step_count(self):
        n = c_size_t()
        check(lib.knhip_executor_step_count(self._h, byref(n)))
        return n.value

    def step_kinds(self):
        kinds = []
        for i in range(self.step_count()):
            k = c_int()
            check(lib.knhip_executor_step_kind(self._h, i, byref(k)))
            kinds.append(STEP_KINDS[k.value])
        return kinds

    def step_work(self, i):
        """(flops, bytes) of one launch of step `i`: multiply-add flops for conv / mat_mul, algorithmic bytes for all."""
        flops, nbytes = c_double(), c_double()
        check(lib.knhip_executor_step_work(self._h, i, byref(flops), byref(nbytes)))
        return flops.value, nbytes.value

    def step_str(self, i):
        return get_string(lib.knhip_executor_step_str, self._h, i)

    def step_source(self, i):
        return get_string(lib.knhip_executor_step_source, self._h, i)

    def fused_source(self):
        """Source of the one kernel that runs the whole plan, "" when the plan is launched step by step."""
        return get_string(lib.knhip_executor_fused_source, self._h)

    def __str__(self):
        return get_string(lib.knhip_executor_str, self._h)


def compile_stats():
    a, b, c = c_size_t(), c_size_t(), c_size_t()
    check(lib.knhip_compile_stats(byref(a), byref(b), byref(c)))
    return {"compiled": a.value, "memory_hits": b.value, "disk_hits": c.value}


class PreparedGraph:
    """kn-runtime/src/lib.rs:104-126 for the `Hip` arm."""

    def __init__(self, executor):
        self.executor = executor

    def eval(self, inputs):
        return self.executor.evaluate(inputs)


class Device:
    """kn-runtime/src/lib.rs:68-102; only the GPU arm exists in this package: there is no CPU execution path."""

    def __init__(self, hip_device):
        self.hip = hip_device

    @staticmethod
    def best():
        if HipDevice.count() == 0:
            raise KnError("no HIP device available and this package has no CPU executor")
        return Device(HipDevice(0))

    @staticmethod
    def parse(text):
        """Device strings as kn-python accepts them (kn-python/src/lib.rs:139-162), with `hip` for `cuda`."""
        if text in ("best", "hip"):
            return Device.best()
        if text.startswith("hip:"):
            return Device(HipDevice(int(text[4:])))
        raise KnError(f"Invalid device string '{text}', expected 'best', 'hip' or 'hip:N'")

    def prepare(self, graph, batch_size):
        return PreparedGraph(HipExecutor(self.hip, graph, batch_size))
