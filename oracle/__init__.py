"""ORACLE - test infrastructure only.

Python loader for `liboracle.so`, the CPU restatement of the reference's `cpu_eval_graph`
(kn-graph/src/cpu.rs:20-23). Only tests, the smoke check and the benchmark's CPU baseline may import this.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, byref, c_char_p, c_int, c_size_t, c_uint8, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")

_NUMPY = [np.float32, np.float64, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64,
          np.bool_, np.float16]


def build():
    """Compile the oracle with gcc (seconds)."""
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    return LIB_PATH


def _load():
    if not os.path.exists(LIB_PATH):
        build()
    lib = ctypes.CDLL(LIB_PATH)
    lib.kn_oracle_last_error.restype = c_char_p
    lib.kn_oracle_eval.argtypes = [POINTER(c_uint8), c_size_t, c_uint64, POINTER(c_void_p), c_size_t, POINTER(c_void_p)]
    lib.kn_oracle_eval.restype = c_int
    lib.kn_oracle_output_count.argtypes = [c_void_p]
    lib.kn_oracle_output_count.restype = c_size_t
    lib.kn_oracle_output_info.argtypes = [c_void_p, c_size_t, POINTER(c_int), POINTER(c_size_t), POINTER(c_size_t),
                                          c_size_t, POINTER(c_void_p), POINTER(c_size_t)]
    lib.kn_oracle_output_info.restype = c_int
    lib.kn_oracle_free.argtypes = [c_void_p]
    lib.kn_oracle_free.restype = None
    return lib


_lib = None


class OracleError(RuntimeError):
    pass


def cpu_eval_graph(graph, batch_size, inputs):
    """`cpu_eval_graph(&graph, batch_size, &inputs) -> Vec<DTensor>`; `graph` is anything with `to_bytes()`
    (or the serialised bytes themselves), inputs are numpy arrays."""
    global _lib
    if _lib is None:
        _lib = _load()
    blob = graph if isinstance(graph, (bytes, bytearray)) else graph.to_bytes()
    buf = (c_uint8 * len(blob)).from_buffer_copy(blob)
    arrays = [np.ascontiguousarray(x) for x in inputs]
    ptrs = (c_void_p * max(len(arrays), 1))(*[a.ctypes.data for a in arrays])
    handle = c_void_p()
    if _lib.kn_oracle_eval(buf, len(blob), batch_size, ptrs, len(arrays), byref(handle)) != 0:
        raise OracleError(_lib.kn_oracle_last_error().decode())
    try:
        outputs = []
        for i in range(_lib.kn_oracle_output_count(handle)):
            dtype, rank, data, nbytes = c_int(), c_size_t(), c_void_p(), c_size_t()
            dims = (c_size_t * 32)()
            if _lib.kn_oracle_output_info(handle, i, byref(dtype), byref(rank), dims, 32, byref(data), byref(nbytes)) != 0:
                raise OracleError("output info failed")
            shape = [dims[k] for k in range(rank.value)]
            dt = np.dtype(_NUMPY[dtype.value])
            if nbytes.value == 0:
                outputs.append(np.zeros(shape, dt))
            else:
                raw = ctypes.string_at(data.value, nbytes.value)
                outputs.append(np.frombuffer(raw, dtype=dt).reshape(shape).copy())
        return outputs
    finally:
        _lib.kn_oracle_free(handle)
