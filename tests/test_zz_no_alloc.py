"""knhip_batched_mat_mul_static, the batched matrix product that allocates nothing: its split-K partial products and
tile counters live in a static device array. Checked through the C ABI against knhip_batched_mat_mul (same kernels, so
bit for bit) and against the oracle, on two calls in a row, the second one smaller, so that what the first call left
in the shared array meets the second."""
import numpy as np
import pytest

from kyanite_amd import (STATIC_SCRATCH_BYTES, DType, DeviceBuffer, HipStream, KnError, batched_mat_mul,
                         batched_mat_mul_static, batched_mat_mul_workspace_bytes, matmul_args)
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs
from test_runtime_shim import _matmul_case

# pairs of (larger, smaller) products; every one needs scratch: dtype, batch, m, n, k
PAIRS = [
    ((DType.F32, 1, 8, 512, 4096), (DType.F32, 1, 8, 256, 1024)),           # split K: partial products
    ((DType.F32, 1, 1024, 8320, 1024), (DType.F32, 1, 8, 512, 4096)),       # tile counters + partial tiles, then split K
    ((DType.F16, 1, 512, 384, 4160), (DType.F16, 1, 33, 33280, 1024)),      # f16 split K, then f16 tail split with counters
]


def _run_pair_member(hip_device, stream, shape, seed):
    dtype, batch, m, n, k = shape
    rng = np.random.default_rng(seed)
    g, a_store, b_store, a_strides, b_strides = _matmul_case(rng, dtype, batch, m, n, k, "mk", "nk")
    np_dtype = a_store.dtype
    a_dev, b_dev = DeviceBuffer.from_array(hip_device, a_store), DeviceBuffer.from_array(hip_device, b_store)
    c_static = DeviceBuffer.from_array(hip_device, np.full((batch, m, n), 7, np_dtype))
    c_plain = DeviceBuffer.from_array(hip_device, np.full((batch, m, n), 9, np_dtype))
    args = matmul_args(dtype, batch, m, n, k, a_dev.ptr, a_strides, b_dev.ptr, b_strides, c_static.ptr, (m * n, n, 1))
    need = batched_mat_mul_workspace_bytes(args)
    assert 0 < need <= STATIC_SCRATCH_BYTES, "the case is meant to use the static scratch"
    print(f"batched_mat_mul_static {dtype.name} {batch}x{m}x{n}x{k}: {need} bytes of scratch", flush=True)
    batched_mat_mul_static(hip_device, stream, args)
    stream.synchronize()
    got = c_static.to_array(np_dtype, (batch, m, n))
    # the existing entry point, on a workspace of the caller's
    args_plain = matmul_args(dtype, batch, m, n, k, a_dev.ptr, a_strides, b_dev.ptr, b_strides, c_plain.ptr, (m * n, n, 1))
    workspace = DeviceBuffer(hip_device, need)
    batched_mat_mul(hip_device, stream, args_plain, workspace)
    stream.synchronize()
    plain = c_plain.to_array(np_dtype, (batch, m, n))
    assert np.array_equal(got.view(np.uint8), plain.view(np.uint8)), f"{shape}: differs from knhip_batched_mat_mul"
    check_outputs(g, 0, [a_store, b_store], cpu_eval_graph(g, 0, [a_store, b_store]), [got],
                  f"batched_mat_mul_static {shape}", PARITY_RECORDS)


@pytest.mark.gpu
@pytest.mark.parametrize("pair", PAIRS, ids=lambda p: f"{p[0][0].name}-{p[0][2]}x{p[0][3]}x{p[0][4]}-then-{p[1][2]}x{p[1][3]}x{p[1][4]}")
def test_two_calls_in_a_row_share_the_static_scratch(pair, hip_device):
    stream = HipStream(hip_device)
    _run_pair_member(hip_device, stream, pair[0], seed=1)
    _run_pair_member(hip_device, stream, pair[1], seed=2)
    # and the larger one again, over what the smaller one left
    _run_pair_member(hip_device, stream, pair[0], seed=3)


@pytest.mark.gpu
def test_products_without_scratch_and_empty_ones(hip_device):
    stream = HipStream(hip_device)
    rng = np.random.default_rng(5)
    g, a_store, b_store, a_strides, b_strides = _matmul_case(rng, DType.F32, 2, 70, 50, 48, "mk", "kn")
    a_dev, b_dev = DeviceBuffer.from_array(hip_device, a_store), DeviceBuffer.from_array(hip_device, b_store)
    c_dev = DeviceBuffer.from_array(hip_device, np.zeros((2, 70, 50), np.float32))
    args = matmul_args(DType.F32, 2, 70, 50, 48, a_dev.ptr, a_strides, b_dev.ptr, b_strides, c_dev.ptr, (3500, 50, 1))
    assert batched_mat_mul_workspace_bytes(args) == 0
    batched_mat_mul_static(hip_device, stream, args)
    stream.synchronize()
    check_outputs(g, 0, [a_store, b_store], cpu_eval_graph(g, 0, [a_store, b_store]), [c_dev.to_array(np.float32, (2, 70, 50))],
                  "batched_mat_mul_static without scratch", PARITY_RECORDS)
    batched_mat_mul_static(hip_device, stream, matmul_args(DType.F32, 0, 70, 50, 48, 0, (0, 48, 1), 0, (0, 50, 1), 0, (0, 50, 1)))
    stream.synchronize()


@pytest.mark.gpu
def test_more_scratch_than_the_static_array_is_refused(hip_device):
    # rejected from the sizes alone, before anything is launched: the operands are never touched
    args = matmul_args(DType.F32, 1, 1536, 1536, 65536, 256, (0, 65536, 1), 256, (0, 1, 65536), 256, (0, 1536, 1))
    assert batched_mat_mul_workspace_bytes(args) > STATIC_SCRATCH_BYTES
    with pytest.raises(KnError, match="static scratch holds"):
        batched_mat_mul_static(hip_device, HipStream(hip_device), args)
