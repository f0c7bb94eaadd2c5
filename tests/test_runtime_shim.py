"""The runtime tier of the C ABI (streams, events, asynchronous copies) and the stand-alone batched matrix product,
driven the way a host language would drive them: the `--skip-io` loop of the reference's profile_net
(kn-cuda-eval/src/bin/profile_net.rs:150-171) with the caller owning uploads, ordering and downloads."""
import numpy as np
import pytest

from kyanite_amd import (DType, DeviceBuffer, Graph, HipExecutor, HipStream, KnError, PinnedMem, batched_mat_mul,
                         batched_mat_mul_workspace_bytes, matmul_args)
from kyanite_amd.configs import build_tiny_mlp
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs


def test_workspace_query_needs_no_device():
    # short K, many tiles: nothing to split; long K on few tiles: partial products; a sparse last round: counters too
    assert batched_mat_mul_workspace_bytes(matmul_args(DType.F32, 1, 1024, 1024, 64, 1, (0, 64, 1), 1, (0, 1024, 1), 1, (0, 1024, 1))) == 0
    split = batched_mat_mul_workspace_bytes(matmul_args(DType.F32, 1, 8, 4096, 4096, 1, (0, 4096, 1), 1, (0, 1, 4096), 1, (0, 4096, 1)))
    assert split == 16 * 8 * 4096 * 4  # 32 tiles of 32 x 128: K in 16 parts
    tail = batched_mat_mul_workspace_bytes(matmul_args(DType.F16, 1, 33, 33280, 1024, 1, (0, 1024, 1), 1, (0, 1, 1024), 1, (0, 33280, 1)))
    assert tail == 256 + 8 * 2 * 64 * 64 * 4  # 8 counters rounded up to 256 bytes, then 8 tiles x 2 parts of 64 x 64 floats
    with pytest.raises(KnError):
        batched_mat_mul_workspace_bytes(matmul_args(DType.I32, 1, 8, 8, 8, 1, (0, 8, 1), 1, (0, 8, 1), 1, (0, 8, 1)))


@pytest.mark.gpu
def test_upload_run_async_event_download(hip_device):
    graph, inputs = build_tiny_mlp(seed=21, batch=8)
    ex = HipExecutor(hip_device, graph, 8, preserve_inputs=True)
    mine = HipStream(hip_device)
    theirs = HipStream.borrowed(hip_device, ex.stream())
    x = inputs[0]
    staging_in, staging_out = PinnedMem(x.nbytes), PinnedMem(8 * 10 * 4)
    out_view = staging_out.array(np.float32, (8, 10))
    for round_ in range(3):
        data = (x * (1.0 + round_)).astype(np.float32)
        staging_in.array(np.float32, x.shape)[...] = data
        out_view[...] = -1.0
        start = mine.record_event()
        # upload on my stream, run on the executor's stream after it, download on mine after the run
        from kyanite_amd._lib import check, lib
        from ctypes import c_void_p
        check(lib.knhip_memcpy_h2d_async(hip_device.index, c_void_p(ex.input_ptr(0)), c_void_p(staging_in.ptr), x.nbytes, mine._h))
        uploaded = mine.record_event()
        theirs.wait_for_event(uploaded)
        ex.run_async()
        ran = theirs.record_event()
        mine.wait_for_event(ran)
        check(lib.knhip_memcpy_d2h_async(hip_device.index, c_void_p(staging_out.ptr), c_void_p(ex.output_ptr(0)), 8 * 10 * 4, mine._h))
        done = mine.record_event()
        done.synchronize()
        assert done.time_elapsed_since(start) >= 0.0 and ran.time_elapsed_since(uploaded) >= 0.0
        got = out_view.copy()
        check_outputs(graph, 8, [data], cpu_eval_graph(graph, 8, [data]), [got], f"run_async with own copies, round {round_}",
                      PARITY_RECORDS)
    mine.synchronize()


@pytest.mark.gpu
def test_device_memory_slices(hip_device):
    """Copies into and between byte ranges of one allocation, with the data and the expected bytes of
    kn-cuda-sys/tests/mem.rs:4-32 (`DevicePtr::offset_bytes`, `copy_linear_from_host`, `copy_linear_from_device`)."""
    from ctypes import c_void_p
    from kyanite_amd._lib import check, lib
    whole = DeviceBuffer(hip_device, 512)
    a, b, c = whole.ptr, whole.ptr + 128, whole.ptr + 256

    def upload(dst, values):
        check(lib.knhip_memcpy_h2d(whole.device, c_void_p(dst), values.ctypes.data, values.nbytes))

    upload(a, np.zeros(512, np.uint8))
    upload(a, np.full(128, 1, np.uint8))
    upload(b, np.full(128, 2, np.uint8))
    check(lib.knhip_memcpy_d2d(whole.device, c_void_p(c), c_void_p(a), 128))
    expected = np.concatenate([np.full(128, v, np.uint8) for v in (1, 2, 1, 0)])
    assert np.array_equal(whole.to_array(np.uint8, (512,)), expected)


def _matmul_case(rng, dtype, batch, m, n, k, a_layout, b_layout, broadcast_b=False):
    """Host arrays laid out as asked plus the strides that address them as A[b, i, k], B[b, k, j]."""
    np_dtype = np.float16 if dtype == DType.F16 else np.float32
    scale = 0.2 if dtype == DType.F16 else 1.0
    a_store = (rng.standard_normal((batch, m, k) if a_layout == "mk" else (batch, k, m)) * scale).astype(np_dtype)
    b_batch = 1 if broadcast_b else batch
    b_store = (rng.standard_normal((b_batch, k, n) if b_layout == "kn" else (b_batch, n, k)) * scale).astype(np_dtype)
    a_strides = (m * k, k, 1) if a_layout == "mk" else (m * k, 1, m)
    b_strides = ((0 if broadcast_b else k * n), n, 1) if b_layout == "kn" else ((0 if broadcast_b else k * n), 1, k)
    g = Graph()
    ga = g.input(list(a_store.shape), dtype)
    gb = g.input(list(b_store.shape), dtype)
    left = ga if a_layout == "mk" else g.permute(ga, [0, 2, 1])
    right = gb if b_layout == "kn" else g.permute(gb, [0, 2, 1])
    if broadcast_b:
        right = g.broadcast(right, [batch, k, n])
    g.output(g.batched_mat_mul(left, right))
    return g, a_store, b_store, a_strides, b_strides


MATMUL_CASES = [
    # dtype, batch, m, n, k, layout of A, layout of B, broadcast B
    (DType.F32, 1, 70, 50, 48, "mk", "kn", False),         # staged kernel, ragged tiles
    (DType.F32, 3, 64, 96, 128, "km", "nk", False),        # transposed left operand, K-contiguous right one
    (DType.F32, 1, 8, 512, 4096, "mk", "nk", False),       # split K: partial products in the workspace
    (DType.F32, 1, 1024, 8320, 256, "mk", "nk", False),    # (direct kernel, more than one round of 128 x 128 tiles)
    (DType.F16, 1, 33, 33280, 1024, "mk", "nk", False),    # tail split: counters and partial tiles in the workspace
    (DType.F16, 2, 200, 136, 192, "mk", "nk", True),       # batch with a broadcast right operand
    (DType.F16, 1, 512, 384, 4160, "mk", "nk", False),     # f16 split K on tall tiles
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", MATMUL_CASES, ids=lambda c: f"{c[0].name}-{c[1]}x{c[2]}x{c[3]}x{c[4]}-{c[5]}-{c[6]}")
def test_batched_mat_mul(case, hip_device):
    dtype, batch, m, n, k, a_layout, b_layout, broadcast_b = case
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    g, a_store, b_store, a_strides, b_strides = _matmul_case(rng, dtype, batch, m, n, k, a_layout, b_layout, broadcast_b)
    print(f"batched_mat_mul {dtype.name} {batch}x{m}x{n}x{k} {a_layout} {b_layout}", flush=True)
    a_dev, b_dev = DeviceBuffer.from_array(hip_device, a_store), DeviceBuffer.from_array(hip_device, b_store)
    np_dtype = a_store.dtype
    c_dev = DeviceBuffer.from_array(hip_device, np.full((batch, m, n), 7, np_dtype))
    args = matmul_args(dtype, batch, m, n, k, a_dev.ptr, a_strides, b_dev.ptr, b_strides, c_dev.ptr, (m * n, n, 1))
    need = batched_mat_mul_workspace_bytes(args)
    # a workspace full of ones: the call has to clear what it relies on
    workspace = DeviceBuffer.from_array(hip_device, np.ones(max(need, 4) // 4 + 64, np.uint32)) if need else None
    stream = HipStream(hip_device)
    expected = cpu_eval_graph(g, 0, [a_store, b_store])
    for round_ in range(2):  # the second call finds the workspace as the first one left it
        batched_mat_mul(hip_device, stream, args, workspace)
        stream.synchronize()
        got = c_dev.to_array(np_dtype, (batch, m, n))
        check_outputs(g, 0, [a_store, b_store], expected, [got], f"batched_mat_mul {case} call {round_}", PARITY_RECORDS)
    if need:
        with pytest.raises(KnError, match="workspace"):
            batched_mat_mul(hip_device, stream, args, None)
