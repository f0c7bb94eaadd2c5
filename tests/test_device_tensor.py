"""DeviceTensor and the stand-alone kernels of the C ABI (knhip_strided_copy, knhip_*_kernel_new / run), the
counterparts of kn-cuda-eval/src/device_tensor.rs:20-169 and src/autokernel/*.rs used outside an executor.

CPU half: constructors check their arguments like the reference's asserts, and every layout compiles for gfx950
without a device. GPU half: copies between arbitrary layouts are bit-exact against numpy indexing; the kernels are
compared with the oracle on the graph that spells the same operation.
"""
import itertools

import numpy as np
import pytest

from kyanite_amd import (DType, DeviceTensor, GatherKernel, Graph, HipStream, KnError, LayernormKernel, ReduceKernel, ReduceOp,
                         ScalarKernel, SoftmaxKernel, StridedShape, batched_mat_mul, batched_mat_mul_workspace_bytes, matmul_args)
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs


# ------------------------------------------------------------------------------------------------------------ CPU half

def test_views_are_stride_and_offset_edits():
    """offset_tensor.rs:52-114 on a tensor without memory behind it (address 1 << 20)"""
    base = DeviceTensor(None, 1 << 20, StridedShape.new_simple([2, 3, 4]), DType.F32)
    assert base.permute([2, 0, 1]).strided_shape == StridedShape([4, 2, 3], [1, 12, 4])
    assert base.view([6, 4]).strided_shape == StridedShape([6, 4], [4, 1])
    with pytest.raises(KnError):
        base.permute([2, 0, 1]).view([8, 3])
    sliced = base.slice(1, 1, 3)
    assert sliced.ptr == (1 << 20) + 4 * 4 and sliced.strided_shape == StridedShape([2, 2, 4], [12, 4, 1])
    stepped = base.slice(2, 1, 3, 2)  # (bounds differ by a multiple of the step, graph.rs SliceRange)
    assert stepped.ptr == (1 << 20) + 4 and stepped.strided_shape == StridedShape([2, 3, 1], [12, 4, 2])
    with pytest.raises(KnError, match="multiple of step"):
        base.slice(2, 1, 4, 2)
    flipped = base.flip(2)
    assert flipped.ptr == (1 << 20) + 3 * 4 and flipped.strided_shape == StridedShape([2, 3, 4], [12, 4, -1])
    assert base.index(0, 1).ptr == (1 << 20) + 48 and base.index(0, 1).strided_shape == StridedShape([3, 4], [4, 1])
    assert base.slice(0, 0, 1).repeat_unary(0, 5).strided_shape == StridedShape([5, 3, 4], [0, 4, 1])
    assert base.index(2, 0).broadcast([7, 2, 3]).strided_shape == StridedShape([7, 2, 3], [0, 12, 4])
    assert base.to_mat_mul_arg() == (1 << 20, (12, 4, 1))
    assert base.permute([0, 2, 1]).to_mat_mul_arg() == (1 << 20, (12, 1, 4))
    with pytest.raises(KnError, match="col- or row-dense"):
        base.slice(2, 0, 4, 2).to_mat_mul_arg()


def test_every_layout_compiles_without_a_device():
    dense = StridedShape.new_simple([3, 4, 5, 6])
    for perm in itertools.permutations(range(4)):
        # stored dense in the permuted order, seen through the inverse permutation: the shape of `dense`, other strides
        src = StridedShape.new_simple([dense.shape[p] for p in perm]).permute([perm.index(a) for a in range(4)])
        assert src.shape == dense.shape
        text, grid, block = ScalarKernel.new_for_shapes(None, "*x0 = *x1;", [dense, src], [DType.F16, DType.F16]).info()
        assert grid >= 1 and block in (64, 256), text
    flipped = StridedShape([3, 4, 5, 6], [120, -30, 6, -1])
    broadcast = StridedShape([3, 4, 5, 6], [0, 6, 0, 1])
    for src in (flipped, broadcast):
        for dtype in (DType.U8, DType.I64, DType.BOOL, DType.F32):
            ScalarKernel.new_for_shapes(None, "*x0 = *x1;", [dense, src], [dtype, dtype])


def test_constructors_refuse_what_the_reference_asserts():
    a = StridedShape.new_simple([4, 6])
    with pytest.raises(KnError, match="should end with ';'"):
        ScalarKernel.new_for_shapes(None, "*x0 = *x1", [a, a], [DType.F32, DType.F32])
    with pytest.raises(KnError, match="shapes differ"):
        ScalarKernel.new_for_shapes(None, "*x0 = *x1;", [a, StridedShape.new_simple([6, 4])], [DType.F32, DType.F32])
    with pytest.raises(KnError, match="broadcast axis"):
        ScalarKernel.new_for_shapes(None, "*x0 = *x1;", [StridedShape([4, 6], [0, 1]), a], [DType.F32, DType.F32])
    with pytest.raises(KnError, match="out of bounds"):
        ReduceKernel(None, ReduceOp.SUM, a, StridedShape.new_simple([4]), [2])
    with pytest.raises(KnError, match="unique"):
        ReduceKernel(None, ReduceOp.SUM, a, StridedShape.new_simple([]), [1, 1])
    with pytest.raises(KnError, match="kept axes"):
        ReduceKernel(None, ReduceOp.SUM, a, StridedShape.new_simple([6]), [1])
    with pytest.raises(KnError, match="shapes differ"):
        SoftmaxKernel(None, a, StridedShape.new_simple([6, 4]), 1)
    with pytest.raises(KnError, match="axis"):
        LayernormKernel(None, a, a, 2, 1e-5)
    with pytest.raises(KnError, match="rank 1"):
        GatherKernel(None, a, a, StridedShape.new_simple([4, 6]), DType.F32, DType.U32, 1)
    with pytest.raises(KnError, match="one entry per index"):
        GatherKernel(None, a, StridedShape.new_simple([3]), StridedShape.new_simple([4, 5]), DType.F32, DType.U32, 1)
    compiled_only = ScalarKernel.new_for_shapes(None, "*x0 = *x1;", [a, a], [DType.F32, DType.F32])
    with pytest.raises(KnError, match="without a device"):
        compiled_only.run(None, [DeviceTensor(None, 256, a, DType.F32), DeviceTensor(None, 512, a, DType.F32)])


# ------------------------------------------------------------------------------------------------------------ GPU half

def _upload(device, array):
    t = DeviceTensor.alloc_simple(device, array.shape, DType.from_numpy(array.dtype))
    t.copy_simple_from_host(array)
    return t


def _random(rng, shape, np_dtype):
    if np_dtype == np.bool_:
        return rng.random(shape) < 0.5
    if np.issubdtype(np_dtype, np.integer):
        info = np.iinfo(np_dtype)
        return rng.integers(info.min, info.max, size=shape, dtype=np_dtype, endpoint=True)
    return rng.standard_normal(shape).astype(np_dtype)


@pytest.mark.gpu
def test_copy_from_all_rank_4_permutes_is_bit_exact(hip_device):
    """the 24 permutations of a rank 4 tensor (graphs.rs:722 has them inside a graph), as source and as destination"""
    rng = np.random.default_rng(5)
    for np_dtype in (np.float32, np.float16, np.uint8):
        host = _random(rng, (5, 7, 6, 9), np_dtype)
        src = _upload(hip_device, host)
        for perm in itertools.permutations(range(4)):
            print(f"copy_from {np_dtype.__name__} permutation {perm}", flush=True)
            permuted = src.permute(list(perm))
            dst = DeviceTensor.alloc_simple(hip_device, permuted.strided_shape.shape, src.dtype)
            dst.copy_from(permuted)  # permuted source -> dense destination
            assert np.array_equal(dst.copy_simple_to_host(), host.transpose(perm)), f"source permuted by {perm}"
            back = DeviceTensor.alloc_simple(hip_device, host.shape, src.dtype)
            back.permute(list(perm)).copy_from(dst)  # dense source -> permuted destination
            assert np.array_equal(back.copy_simple_to_host(), host), f"destination permuted by {perm}"


@pytest.mark.gpu
@pytest.mark.parametrize("np_dtype", [np.float32, np.float16, np.int64, np.uint8, np.bool_, np.float64, np.int16])
def test_copy_from_flipped_sliced_and_broadcast_sources(hip_device, np_dtype):
    rng = np.random.default_rng(6)
    host = _random(rng, (6, 10, 12), np_dtype)
    src = _upload(hip_device, host)
    cases = {
        "flip axis 2": (src.flip(2), host[:, :, ::-1]),
        "flip axes 0 and 1": (src.flip(0).flip(1), host[::-1, ::-1]),
        "slice with step": (src.slice(1, 1, 10, 3), host[:, 1:10:3]),
        "slice of a flip": (src.flip(2).slice(2, 2, 12, 2), host[:, :, ::-1][:, :, 2:12:2]),
        "broadcast": (src.index(1, 4).view([6, 1, 12]).broadcast([6, 5, 12]), np.broadcast_to(host[:, 4:5], (6, 5, 12))),
        "index then permute": (src.index(0, 3).permute([1, 0]), host[3].T),
    }
    for name, (view, expected) in cases.items():
        print(f"copy_from {np_dtype.__name__} {name}", flush=True)
        dst = DeviceTensor.alloc_simple(hip_device, view.strided_shape.shape, src.dtype)
        dst.copy_from(view)
        assert np.array_equal(dst.copy_simple_to_host(), expected), name
        assert np.array_equal(view.copy_to_host_staged(), expected), f"{name}, copy_to_host_staged"
    # a flipped, strided destination; the rest of the buffer keeps its contents
    target = _upload(hip_device, host)
    piece = _random(rng, (6, 3, 12), np_dtype)
    target.flip(1).slice(1, 0, 9, 3).copy_from(_upload(hip_device, piece))
    expected = host.copy()
    expected[:, ::-1][:, 0:9:3] = piece
    assert np.array_equal(target.copy_simple_to_host(), expected)
    # the same through the host: copy_from_host_staged into a view
    target2 = _upload(hip_device, host)
    piece2 = _random(rng, (3, 6, 10), np_dtype)
    target2.permute([2, 0, 1]).slice(0, 0, 12, 4).copy_from_host_staged(piece2)
    expected2 = host.copy()
    expected2.transpose(2, 0, 1)[0:12:4] = piece2
    assert np.array_equal(target2.copy_simple_to_host(), expected2)


@pytest.mark.gpu
def test_copy_from_same_dense_layout_is_one_linear_copy(hip_device):
    """both sides permuted (and flipped) alike: dense strides that match, the memcpy branch of device_tensor.rs:115-118"""
    rng = np.random.default_rng(7)
    host = rng.standard_normal((8, 5, 16)).astype(np.float32)
    src = _upload(hip_device, host)
    dst = DeviceTensor.alloc_simple(hip_device, host.shape, DType.F32)
    dst.permute([2, 0, 1]).flip(1).copy_from(src.permute([2, 0, 1]).flip(1))
    assert np.array_equal(dst.copy_simple_to_host(), host)
    clone = src.permute([1, 0, 2]).deep_clone()
    assert clone.strided_shape.has_simple_strides() and np.array_equal(clone.copy_simple_to_host(), host.transpose(1, 0, 2))
    empty = DeviceTensor.alloc_simple(hip_device, [0, 4], DType.F32)
    empty.copy_from(DeviceTensor.alloc_simple(hip_device, [0, 4], DType.F32))
    with pytest.raises(KnError, match="same dtype"):
        dst.copy_from(DeviceTensor.alloc_simple(hip_device, host.shape, DType.F16))
    with pytest.raises(KnError, match="shapes differ"):
        dst.copy_from(src.permute([1, 0, 2]))


@pytest.mark.gpu
def test_scalar_kernel_on_strided_operands(hip_device):
    rng = np.random.default_rng(8)
    stream = HipStream(hip_device)
    a, b = rng.standard_normal((32, 48)).astype(np.float32), rng.standard_normal((48,)).astype(np.float32)
    ta, tb = _upload(hip_device, a.T.copy()).permute([1, 0]), _upload(hip_device, b).view([1, 48]).broadcast([32, 48])
    out = DeviceTensor.alloc_simple(hip_device, [32, 48], DType.F32)
    kernel = ScalarKernel.new_for_shapes(hip_device, "*x0 = *x1 * *x2 + 1.5f;", [out.strided_shape, ta.strided_shape, tb.strided_shape],
                                         [DType.F32] * 3)
    kernel.run(stream, [out, ta, tb])
    stream.synchronize()
    assert np.array_equal(out.copy_simple_to_host(), a * b[None, :] + np.float32(1.5))
    with pytest.raises(KnError, match="does not match"):
        kernel.run(stream, [out, _upload(hip_device, a), tb])  # dense where the kernel was built for transposed storage
    # integers with wrap-around and a result of another type
    x = rng.integers(0, 255, size=(1000,), dtype=np.uint8)
    tx, wide = _upload(hip_device, x), DeviceTensor.alloc_simple(hip_device, [1000], DType.I32)
    ScalarKernel.new_for_shapes(hip_device, "*x0 = (int) *x1 * 3 - 7;", [wide.strided_shape, tx.strided_shape],
                                [DType.I32, DType.U8]).run(stream, [wide, tx])
    stream.synchronize()
    assert np.array_equal(wide.copy_simple_to_host(), x.astype(np.int32) * 3 - 7)
    # halves are floats inside the operation and are rounded once at the store
    h = rng.standard_normal((64, 40)).astype(np.float16)
    th, ho = _upload(hip_device, h), DeviceTensor.alloc_simple(hip_device, [64, 40], DType.F16)
    ScalarKernel.new_for_shapes(hip_device, "*x0 = *x1 * 0.5f + 1.0f;", [ho.strided_shape, th.strided_shape],
                                [DType.F16, DType.F16]).run(stream, [ho, th])
    stream.synchronize()
    assert np.array_equal(ho.copy_simple_to_host(), (h.astype(np.float32) * np.float32(0.5) + np.float32(1.0)).astype(np.float16))


def _oracle(build, inputs):
    g = Graph()
    build(g, [g.input(list(x.shape), DType.from_numpy(x.dtype)) for x in inputs])
    return g, cpu_eval_graph(g, 0, inputs)


@pytest.mark.gpu
def test_reduce_softmax_layernorm_kernels_against_the_oracle(hip_device):
    rng = np.random.default_rng(9)
    stream = HipStream(hip_device)
    x = rng.standard_normal((24, 50, 33)).astype(np.float32)
    tx = _upload(hip_device, x)

    for op, axes in ((ReduceOp.SUM, [2]), (ReduceOp.MAX, [0, 2]), (ReduceOp.MEAN, [1]), (ReduceOp.MIN, [0]), (ReduceOp.PROD, [2])):
        print(f"reduce kernel {op.name} over {axes}", flush=True)
        kept = [d for a, d in enumerate(x.shape) if a not in axes]
        out = DeviceTensor.alloc_simple(hip_device, kept, DType.F32)
        ReduceKernel(hip_device, op, tx.strided_shape, out.strided_shape, axes).run(stream, tx, out)
        stream.synchronize()
        g, expected = _oracle(lambda g, v: g.output(g.reduce(v[0], axes, op)), [x])
        check_outputs(g, 0, [x], expected, [out.copy_simple_to_host()], f"reduce kernel {op.name} {axes}", PARITY_RECORDS)

    # a permuted input and a strided output: softmax along what is axis 0 of the view
    view = tx.permute([1, 0, 2])
    out = DeviceTensor.alloc_simple(hip_device, [50, 24, 33], DType.F32)
    SoftmaxKernel(hip_device, view.strided_shape, out.strided_shape, 0, 0.75).run(stream, view, out)
    stream.synchronize()
    xp = np.ascontiguousarray(x.transpose(1, 0, 2))
    g, expected = _oracle(lambda g, v: g.output(g.softmax(g.mul(v[0], g.scalar(0.75)), 0)), [xp])
    check_outputs(g, 0, [xp], expected, [out.copy_simple_to_host()], "softmax kernel, scaled, permuted input", PARITY_RECORDS)

    y = rng.standard_normal(x.shape).astype(np.float32)
    ty, out = _upload(hip_device, y), DeviceTensor.alloc_simple(hip_device, x.shape, DType.F32)
    LayernormKernel(hip_device, tx.strided_shape, out.strided_shape, 2, 1e-5, 0.5, 2.0, 3.0).run(stream, tx, ty, out)
    stream.synchronize()
    g, expected = _oracle(lambda g, v: g.output(g.mul(g.layernorm(g.add(g.mul(v[0], g.scalar(0.5)), g.mul(v[1], g.scalar(2.0))), 2, 1e-5),
                                                       g.scalar(3.0))), [x, y])
    check_outputs(g, 0, [x, y], expected, [out.copy_simple_to_host()], "layernorm kernel, two inputs", PARITY_RECORDS)
    plain = LayernormKernel(hip_device, tx.strided_shape, out.strided_shape, 1, 1e-3)
    plain.run(stream, tx, None, out)
    stream.synchronize()
    g, expected = _oracle(lambda g, v: g.output(g.layernorm(v[0], 1, 1e-3)), [x])
    check_outputs(g, 0, [x], expected, [out.copy_simple_to_host()], "layernorm kernel, one input", PARITY_RECORDS)


@pytest.mark.gpu
def test_gather_kernel_and_mat_mul_arg(hip_device):
    rng = np.random.default_rng(10)
    stream = HipStream(hip_device)
    x = rng.standard_normal((6, 40, 9)).astype(np.float16)
    idx = np.array([3, 39, 0, 40, 7, 7, 1000], np.uint32)  # 40 and 1000 are out of range: zeros (gather.cu:46-49)
    tx, ti = _upload(hip_device, x), _upload(hip_device, idx)
    out = DeviceTensor.alloc_simple(hip_device, [6, 7, 9], DType.F16)
    GatherKernel(hip_device, tx.strided_shape, ti.strided_shape, out.strided_shape, DType.F16, DType.U32, 1).run(stream, tx, ti, out)
    stream.synchronize()
    expected = np.where((idx < 40)[None, :, None], x[:, np.minimum(idx, 39)], np.float16(0))
    assert np.array_equal(out.copy_simple_to_host(), expected)

    # to_mat_mul_arg feeds the stand-alone product: A [2, 16, 24] row-major, B stored as [2, 20, 24] and read transposed
    a, b = rng.standard_normal((2, 16, 24)).astype(np.float32), rng.standard_normal((2, 20, 24)).astype(np.float32)
    ta, tb = _upload(hip_device, a), _upload(hip_device, b).permute([0, 2, 1])
    tc = DeviceTensor.alloc_simple(hip_device, [2, 16, 20], DType.F32)
    (pa, sa), (pb, sb), (pc, sc) = ta.to_mat_mul_arg(), tb.to_mat_mul_arg(), tc.to_mat_mul_arg()
    args = matmul_args(DType.F32, 2, 16, 20, 24, pa, sa, pb, sb, pc, sc)
    assert batched_mat_mul_workspace_bytes(args) == 0
    batched_mat_mul(hip_device, stream, args)
    stream.synchronize()
    g, expected = _oracle(lambda g, v: g.output(g.batched_mat_mul(v[0], g.permute(v[1], [0, 2, 1]))), [a, b])
    check_outputs(g, 0, [a, b], expected, [tc.copy_simple_to_host()], "to_mat_mul_arg", PARITY_RECORDS)
