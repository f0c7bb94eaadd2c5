"""Loads libknhip.so and declares the C ABI of include/knhip.h for ctypes.

There is no fallback: if the library is missing (run `python kyanite_amd/build.py`) importing fails loudly.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_uint8, c_uint32, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libknhip.so")


class KnError(RuntimeError):
    """Raised where the reference would panic."""


class SizeT(Structure):
    _fields_ = [("fixed_factor", c_uint64), ("batch_exp", c_uint32)]


class ValueInfoT(Structure):
    _fields_ = [
        ("dtype", c_int), ("op", c_int), ("sub_op", c_int), ("cast_dtype", c_int),
        ("rank", c_size_t), ("operand_count", c_size_t), ("axis_count", c_size_t), ("non_output_uses", c_size_t),
        ("slice_start", c_size_t), ("slice_end", c_size_t), ("slice_step", c_size_t),
        ("eps", c_float), ("is_hidden", c_int),
    ]


class OptimizerSettingsT(Structure):
    _fields_ = [("optimize", c_int), ("force_bias_through_conv", c_int), ("fuse_layernorm", c_int), ("div_to_mul", c_int)]


class ProfileT(Structure):
    _fields_ = [("per_kind", c_float * 7), ("total_cpu", c_float), ("total_gpu", c_float), ("timing_overhead", c_float),
                ("step_count", c_size_t)]


class MatmulArgsT(Structure):
    _fields_ = [("dtype", c_int), ("batch", c_int), ("m", c_int), ("n", c_int), ("k", c_int),
                ("a", c_void_p), ("a_batch_stride", c_int64), ("a_row_stride", c_int64), ("a_col_stride", c_int64),
                ("b", c_void_p), ("b_batch_stride", c_int64), ("b_row_stride", c_int64), ("b_col_stride", c_int64),
                ("c", c_void_p), ("c_batch_stride", c_int64), ("c_row_stride", c_int64), ("c_col_stride", c_int64)]


class ExecutorOptionsT(Structure):
    _fields_ = ([("struct_bytes", c_size_t)] +
                [(name, c_int) for name in (
                    "plan_only", "preserve_inputs", "step_by_step", "fuse_attention", "fuse_gated_matmul", "group_matmuls", "pack_matmul_constants",
                    "pointwise_conv_as_matmul", "join_elementwise", "split_reduce", "tiled_transpose", "split_conv_channels",
                    "plane_conv_any_width", "direct_gemm", "split_k", "tail_split", "dot_products")] +
                [("streaming_bytes", c_uint64), ("mapped_io_bytes", c_uint64), ("stream_weights_bytes", c_uint64)])


class TensorT(Structure):
    _fields_ = [("ptr", c_void_p), ("dtype", c_int), ("rank", c_size_t), ("shape", POINTER(c_size_t)), ("strides", POINTER(c_int64))]


class MemUsageT(Structure):
    _fields_ = [("dedicated_bytes", c_size_t), ("shared_bytes", c_size_t), ("zero_bytes", c_size_t),
                ("hypo_shared_bytes_peak", c_size_t), ("hypo_shared_bytes_total", c_size_t), ("arena_bytes", c_size_t)]


V = c_uint32
PV = POINTER(V)
PS = POINTER(SizeT)
PZ = POINTER(c_size_t)
G = c_void_p
E = c_void_p

# name -> argument types; every function returns int except the three noted below
SIGNATURES = {
    "knhip_device_count": [POINTER(c_int)],
    "knhip_device_name": [c_int, c_char_p, c_size_t, PZ],
    "knhip_malloc": [c_int, c_size_t, POINTER(c_void_p)],
    "knhip_free": [c_int, c_void_p],
    "knhip_memcpy_h2d": [c_int, c_void_p, c_void_p, c_size_t],
    "knhip_memcpy_d2h": [c_int, c_void_p, c_void_p, c_size_t],
    "knhip_memcpy_d2d": [c_int, c_void_p, c_void_p, c_size_t],
    "knhip_host_alloc": [c_size_t, POINTER(c_void_p)],
    "knhip_host_free": [c_void_p],
    "knhip_device_synchronize": [c_int],
    "knhip_stream_create": [c_int, POINTER(c_void_p)],
    "knhip_stream_destroy": [c_int, c_void_p],
    "knhip_stream_synchronize": [c_int, c_void_p],
    "knhip_stream_wait_event": [c_int, c_void_p, c_void_p],
    "knhip_event_create": [c_int, POINTER(c_void_p)],
    "knhip_event_destroy": [c_int, c_void_p],
    "knhip_event_record": [c_int, c_void_p, c_void_p],
    "knhip_event_synchronize": [c_int, c_void_p],
    "knhip_event_elapsed_seconds": [c_int, c_void_p, c_void_p, POINTER(c_float)],
    "knhip_memcpy_h2d_async": [c_int, c_void_p, c_void_p, c_size_t, c_void_p],
    "knhip_memcpy_d2h_async": [c_int, c_void_p, c_void_p, c_size_t, c_void_p],
    "knhip_memcpy_d2d_async": [c_int, c_void_p, c_void_p, c_size_t, c_void_p],
    "knhip_batched_mat_mul_workspace_bytes": [POINTER(MatmulArgsT), PZ],
    "knhip_batched_mat_mul": [c_int, c_void_p, POINTER(MatmulArgsT), c_void_p, c_size_t],
    "knhip_batched_mat_mul_static": [c_int, c_void_p, POINTER(MatmulArgsT)],
    "knhip_static_scratch_prepare": [c_int],
    "knhip_strided_copy": [c_int, c_void_p, POINTER(TensorT), POINTER(TensorT)],
    "knhip_scalar_kernel_new": [c_int, c_char_p, POINTER(TensorT), c_size_t, POINTER(c_void_p)],
    "knhip_reduce_kernel_new": [c_int, c_int, POINTER(TensorT), POINTER(TensorT), PZ, c_size_t, POINTER(c_void_p)],
    "knhip_softmax_kernel_new": [c_int, POINTER(TensorT), POINTER(TensorT), c_size_t, c_float, POINTER(c_void_p)],
    "knhip_layernorm_kernel_new": [c_int, POINTER(TensorT), POINTER(TensorT), c_size_t, c_float, c_float, c_float, c_float,
                                   POINTER(c_void_p)],
    "knhip_gather_kernel_new": [c_int, POINTER(TensorT), POINTER(TensorT), POINTER(TensorT), c_size_t, POINTER(c_void_p)],
    "knhip_kernel_run": [c_void_p, c_void_p, POINTER(c_void_p), c_size_t],
    "knhip_kernel_info": [c_void_p, c_char_p, c_size_t, PZ, POINTER(ctypes.c_uint), POINTER(ctypes.c_uint)],
    "knhip_graph_new": [POINTER(G)],
    "knhip_graph_clone": [G, POINTER(G)],
    "knhip_graph_deserialize": [POINTER(c_uint8), c_size_t, POINTER(G)],
    "knhip_graph_serialize": [G, POINTER(c_uint8), c_size_t, PZ],
    "knhip_graph_str": [G, c_char_p, c_size_t, PZ],
    "knhip_graph_input": [G, PS, c_size_t, c_int, PV],
    "knhip_graph_constant": [G, PS, c_size_t, c_int, c_void_p, c_size_t, PV],
    "knhip_graph_view": [G, V, PS, c_size_t, PV],
    "knhip_graph_broadcast": [G, V, PS, c_size_t, PV],
    "knhip_graph_repeat_unary": [G, V, c_size_t, SizeT, PV],
    "knhip_graph_flatten": [G, V, c_size_t, PV],
    "knhip_graph_permute": [G, V, PZ, c_size_t, PV],
    "knhip_graph_slice": [G, V, c_size_t, c_size_t, c_size_t, c_size_t, PV],
    "knhip_graph_index": [G, V, c_size_t, c_size_t, PV],
    "knhip_graph_flip": [G, V, c_size_t, PV],
    "knhip_graph_repeat": [G, V, c_size_t, SizeT, c_int, PV],
    "knhip_graph_gather": [G, V, c_size_t, V, PV],
    "knhip_graph_concat": [G, PV, c_size_t, c_size_t, PS, c_size_t, c_int, PV],
    "knhip_graph_pad": [G, V, PZ, c_size_t, V, PV],
    "knhip_graph_conv": [G, V, V, c_size_t, c_size_t, c_size_t, c_size_t, PV],
    "knhip_graph_linear": [G, V, V, PV],
    "knhip_graph_mat_mul": [G, V, V, PV],
    "knhip_graph_batched_mat_mul": [G, V, V, PV],
    "knhip_graph_softmax": [G, V, c_size_t, PV],
    "knhip_graph_layernorm": [G, V, c_size_t, c_float, PV],
    "knhip_graph_reduce": [G, V, PZ, c_size_t, c_int, PV],
    "knhip_graph_clamp": [G, V, c_void_p, c_void_p, PV],
    "knhip_graph_relu": [G, V, PV],
    "knhip_graph_unary": [G, c_int, c_int, V, PV],
    "knhip_graph_binary": [G, c_int, V, V, PV],
    "knhip_graph_call": [G, G, PV, c_size_t, PV, c_size_t, PZ],
    "knhip_graph_output": [G, V],
    "knhip_graph_set_debug_id": [G, V, c_char_p],
    "knhip_graph_value_count": [G, PZ],
    "knhip_graph_inputs": [G, PV, c_size_t, PZ],
    "knhip_graph_outputs": [G, PV, c_size_t, PZ],
    "knhip_graph_value_info": [G, V, POINTER(ValueInfoT)],
    "knhip_graph_value_shape": [G, V, PS, c_size_t],
    "knhip_graph_value_operands": [G, V, PV, c_size_t],
    "knhip_graph_value_axes": [G, V, PZ, c_size_t],
    "knhip_graph_value_constant": [G, V, POINTER(c_void_p), PZ],
    "knhip_graph_as_single_const": [G, V, POINTER(c_int), c_void_p],
    "knhip_graph_as_const": [G, V, POINTER(c_int), c_void_p, c_size_t, PZ],
    "knhip_graph_infer_batch_size": [G, PZ, PZ, c_size_t, POINTER(c_int), POINTER(c_int), POINTER(c_uint64)],
    "knhip_optimizer_settings_default": [POINTER(OptimizerSettingsT)],
    "knhip_graph_optimize": [G, POINTER(OptimizerSettingsT), POINTER(G)],
    "knhip_executor_options_default": [POINTER(ExecutorOptionsT)],
    "knhip_executor_new": [c_int, G, c_size_t, POINTER(ExecutorOptionsT), POINTER(E)],
    "knhip_executor_new_from_blob": [c_int, POINTER(c_uint8), c_size_t, c_size_t, POINTER(ExecutorOptionsT), POINTER(E)],
    "knhip_executor_io_count": [E, PZ, PZ],
    "knhip_executor_io_info": [E, c_int, c_size_t, POINTER(c_int), PZ, PZ, c_size_t],
    "knhip_executor_evaluate": [E, POINTER(c_void_p), PZ, c_size_t, POINTER(c_void_p), PZ, c_size_t],
    "knhip_executor_run_async": [E],
    "knhip_executor_synchronize": [E],
    "knhip_executor_time_runs": [E, c_size_t, POINTER(c_float)],
    "knhip_executor_input_ptr": [E, c_size_t, POINTER(c_void_p)],
    "knhip_executor_output_ptr": [E, c_size_t, POINTER(c_void_p)],
    "knhip_executor_stream": [E, POINTER(c_void_p)],
    "knhip_executor_set_profile": [E, c_int],
    "knhip_executor_last_profile": [E, POINTER(c_int), POINTER(ProfileT)],
    "knhip_executor_profile_step_seconds": [E, POINTER(c_float), c_size_t],
    "knhip_executor_profile_str": [E, c_char_p, c_size_t, PZ],
    "knhip_executor_mem_usage": [E, POINTER(MemUsageT)],
    "knhip_executor_step_count": [E, PZ],
    "knhip_executor_step_kind": [E, c_size_t, POINTER(c_int)],
    "knhip_executor_step_str": [E, c_size_t, c_char_p, c_size_t, PZ],
    "knhip_executor_set_graph_mode": [E, c_int],
    "knhip_executor_step_work": [E, c_size_t, POINTER(c_double), POINTER(c_double)],
    "knhip_executor_step_source": [E, c_size_t, c_char_p, c_size_t, PZ],
    "knhip_executor_fused_source": [E, c_char_p, c_size_t, PZ],
    "knhip_executor_str": [E, c_char_p, c_size_t, PZ],
    "knhip_strided_flags": [PZ, POINTER(c_int64), c_size_t, POINTER(c_int), POINTER(c_int)],
    "knhip_strided_view": [PZ, POINTER(c_int64), c_size_t, PZ, c_size_t, POINTER(c_int), POINTER(c_int64)],
    "knhip_strided_slice": [PZ, POINTER(c_int64), c_size_t, c_size_t, c_size_t, c_size_t, c_size_t, PZ, POINTER(c_int64)],
    "knhip_compile_stats": [PZ, PZ, PZ],
}
# functions that do not return a status
SPECIAL = {
    "knhip_last_error": ([], c_char_p),
    "knhip_graph_free": ([G], None),
    "knhip_executor_free": ([E], None),
    "knhip_kernel_free": ([c_void_p], None),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python kyanite_amd/build.py` "
                          "(there is no fallback implementation)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    for name, (argtypes, restype) in SPECIAL.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    return lib


lib = _load()


def check(status):
    if status != 0:
        raise KnError(lib.knhip_last_error().decode("utf-8", "replace"))


def get_string(fn, *args):
    needed = c_size_t(0)
    check(fn(*args, None, 0, ctypes.byref(needed)))
    buf = ctypes.create_string_buffer(needed.value)
    check(fn(*args, buf, needed.value, ctypes.byref(needed)))
    return buf.value.decode("utf-8", "replace")
