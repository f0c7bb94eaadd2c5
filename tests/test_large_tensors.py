"""Tensors of more than 2^31 elements, and buffers that lie past the first 4 GiB of device memory: the generated
kernels switch to 64 bit indices there, which no other test reaches. The reference holds one such case,
`layernorm_huge` (kn-cuda-eval/tests/root/slow.rs:12-31, ignored by default there); it is restated here with its
shape and its 4 GiB of ballast, next to one case per kernel generator.

The executors are driven through copies into their input buffers, `run_async` and device-to-host copies of byte
ranges, the way a caller that owns its buffers does, so that neither page-locked staging nor host arrays of several GiB
are needed: an input is one block of 98 MB uploaded again and again until the tensor is full (the block is 12007 rows
of 4096 halves long, a prime number of rows, so no power-of-two stride meets equal data), and what a value must be
follows from its flat index. What comes back is compared exactly (integer work, data movement, max) or, for float
rows, against the oracle on the very rows that were fetched (rows of a softmax or of a sum along the row do not depend
on each other).
"""
from ctypes import c_void_p

import numpy as np
import pytest

from kyanite_amd import DType, DeviceBuffer, Graph, HipExecutor, ReduceOp
from kyanite_amd._lib import check, lib
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

pytestmark = pytest.mark.gpu

PAST_I32 = 1 << 31
BLOCK_ROWS, BLOCK_WIDTH = 12007, 4096
BLOCK = BLOCK_ROWS * BLOCK_WIDTH  # halves; twice as many bytes


@pytest.fixture(scope="module")
def block():
    return np.random.default_rng(1).standard_normal(BLOCK).astype(np.float16)


@pytest.fixture(scope="module")
def block32():
    return np.random.default_rng(2).standard_normal(BLOCK // 2).astype(np.float32)


def _fill_input(ex, index, piece, count):
    """input `index` := `piece` repeated over `count` elements: one upload, then device-to-device copies that double
    what is filled"""
    base, item = ex.input_ptr(index), piece.itemsize
    filled = min(piece.size, count)
    check(lib.knhip_memcpy_h2d(ex.device, c_void_p(base), piece.ctypes.data, filled * item))
    while filled < count:
        step = min(filled, count - filled)
        check(lib.knhip_memcpy_d2d(ex.device, c_void_p(base + filled * item), c_void_p(base), step * item))
        filled += step
    return piece


def _stretch(piece, first, count):
    """elements `first .. first + count` of the repeated piece"""
    return piece[(first + np.arange(count, dtype=np.int64)) % piece.size]


def _run(ex):
    ex.run_async()
    ex.synchronize()


def _fetch(ex, output, first_element, count, dtype):
    """`count` elements of output `output`, starting at flat element `first_element`."""
    out = np.empty(count, dtype)
    check(lib.knhip_memcpy_d2h(ex.device, out.ctypes.data, c_void_p(ex.output_ptr(output) + first_element * out.itemsize), out.nbytes))
    return out


def test_elementwise_past_2_31_elements(hip_device, block):
    n = PAST_I32 + 4096
    g = Graph()
    x = g.input([n], DType.U8)
    g.output(g.add(x, g.scalar(3, DType.U8)))
    assert "idx=64" in HipExecutor(0, g, 0, plan_only=True).step_str(0)
    ex = HipExecutor(hip_device, g, 0)
    piece = _fill_input(ex, 0, block.view(np.uint8), n)
    _run(ex)
    expected = piece + np.uint8(3)
    for first in range(0, n, piece.size):  # the whole output, one period of the input at a time
        count = min(piece.size, n - first)
        assert np.array_equal(_fetch(ex, 0, first, count, np.uint8), expected[:count]), f"from element {first}"


def test_transposing_copy_past_2_31_elements(hip_device, block):
    rows, cols = 32769, 65536
    g = Graph()
    x = g.input([rows, cols], DType.U8)
    g.output(g.add(g.permute(x, [1, 0]), g.scalar(1, DType.U8)))
    assert "idx=64" in HipExecutor(0, g, 0, plan_only=True).step_str(0)
    ex = HipExecutor(hip_device, g, 0)
    piece = _fill_input(ex, 0, block.view(np.uint8), rows * cols)
    _run(ex)
    r = np.arange(rows, dtype=np.int64)
    for c0 in [0, 64, 4096, 32704, 32768, 32832, 65408, 65472]:  # 64 output rows each, around every power of two
        c = np.arange(c0, c0 + 64, dtype=np.int64)
        expected = piece[(r[None, :] * cols + c[:, None]) % piece.size] + np.uint8(1)
        got = _fetch(ex, 0, c0 * rows, 64 * rows, np.uint8).reshape(64, rows)
        assert np.array_equal(got, expected), f"output rows {c0}.."


def test_gather_from_a_table_past_2_31_elements(hip_device, block):
    n = PAST_I32 + 64
    g = Graph()
    table = g.input([n], DType.U8)
    indices = g.input([1000], DType.I64)
    g.output(g.gather(table, 0, indices))
    ex = HipExecutor(hip_device, g, 0)
    piece = _fill_input(ex, 0, block.view(np.uint8), n)
    rng = np.random.default_rng(4)
    picks = np.concatenate([rng.integers(0, n, 988), [0, n - 1, PAST_I32 - 1, PAST_I32, PAST_I32 + 1, n - 2, 1, 2, 3, 4, n, -1]]).astype(np.int64)
    ex.upload_input(1, picks)
    _run(ex)
    inside = (picks >= 0) & (picks < n)  # an index outside the table reads as 0
    assert np.array_equal(_fetch(ex, 0, 0, 1000, np.uint8), np.where(inside, piece[picks % piece.size], 0).astype(np.uint8))


def _row_samples(rows):
    """the first and the last rows, and rows either side of the place where a 32 bit element index would wrap"""
    return [0, 1, 2, 3, rows // 2 - 1, rows // 2, rows // 2 + 1, rows - 4, rows - 3, rows - 2, rows - 1]


def test_softmax_rows_past_2_31_elements(hip_device, block):
    rows, width = (1 << 21) + 8, 1024
    g = Graph()
    x = g.input([rows, width], DType.F16)
    g.output(g.softmax(x, 1))
    ex = HipExecutor(hip_device, g, 0)
    _fill_input(ex, 0, block, rows * width)
    _run(ex)
    picked = _row_samples(rows)
    got = np.stack([_fetch(ex, 0, r * width, width, np.float16) for r in picked])
    sample = np.ascontiguousarray(block.reshape(-1, width)[[r % (BLOCK // width) for r in picked]])
    small = Graph()
    sx = small.input([len(picked), width], DType.F16)
    small.output(small.softmax(sx, 1))
    check_outputs(small, 0, [sample], cpu_eval_graph(small, 0, [sample]), [got], "softmax rows of a 4 GiB tensor", PARITY_RECORDS)


@pytest.mark.parametrize("two_steps", [True, False])
def test_softmax_over_a_middle_axis_past_2_31_elements(hip_device, block, two_steps):
    """the normalised axis is not the contiguous one and no workgroup can hold a column: as a reduction to (maximum,
    1 / sum of exponentials) and an elementwise kernel, or (with that plan switched off) the row kernel with lanes
    across columns that reads every column again per pass"""
    batch, length, width = 3, 700, (1 << 20) + 8
    g = Graph()
    x = g.input([batch, length, width], DType.F16)
    g.output(g.softmax(x, 1))
    options = {} if two_steps else {"split_reduce": False}
    plan = HipExecutor(0, g, 0, plan_only=True, **options)
    if two_steps:
        assert plan.step_count() == 2 and "maximum and sum of exponentials" in plan.step_str(0)
        assert all("typedef long long idx_t" in plan.step_source(i) for i in range(2))
    else:
        assert "columns" in plan.step_str(0) and "typedef long long idx_t" in plan.step_source(0)
    ex = HipExecutor(hip_device, g, 0, **options)
    _fill_input(ex, 0, block, batch * length * width)
    _run(ex)
    # 16 neighbouring columns at a time: the first and the last of every batch entry, and either side of the place
    # where a 32 bit element index would wrap (flat element 2^31 lies in batch entry 2)
    wrap_row, wrap_col = divmod(PAST_I32 - 2 * length * width, width)
    picked = [(0, 0), (0, width - 16), (1, 524288), (2, min(wrap_col, width - 16)), (2, width - 16)]
    small = Graph()
    small.output(small.softmax(small.input([len(picked), length, 16], DType.F16), 1))
    sample = np.empty((len(picked), length, 16), np.float16)
    got = np.empty_like(sample)
    for i, (b, col) in enumerate(picked):
        for row in range(length):
            first = (b * length + row) * width + col
            sample[i, row] = _stretch(block, first, 16)
            got[i, row] = _fetch(ex, 0, first, 16, np.float16)
    check_outputs(small, 0, [sample], cpu_eval_graph(small, 0, [sample]), [got], "softmax over the middle axis of a 4.4 GB tensor",
                  PARITY_RECORDS)


def test_reduce_past_2_31_elements(hip_device, block):
    rows, width = (1 << 19) + 1, BLOCK_WIDTH
    g = Graph()
    x = g.input([rows, width], DType.F16)
    g.output(g.reduce(x, [1], ReduceOp.SUM))
    g.output(g.reduce(x, [0], ReduceOp.MAX))
    ex = HipExecutor(hip_device, g, 0)
    _fill_input(ex, 0, block, rows * width)
    _run(ex)
    picked = _row_samples(rows)
    sums = np.array([_fetch(ex, 0, r, 1, np.float16)[0] for r in picked])
    by_row = block.reshape(BLOCK_ROWS, width)
    sample = np.ascontiguousarray(by_row[[r % BLOCK_ROWS for r in picked]])
    small = Graph()
    sx = small.input([len(picked), width], DType.F16)
    small.output(small.reduce(sx, [1], ReduceOp.SUM))
    check_outputs(small, 0, [sample], cpu_eval_graph(small, 0, [sample]), [sums], "row sums of a 4 GiB tensor", PARITY_RECORDS)
    # every row of the block occurs (524289 rows, period 12007), so a column's maximum is the block's
    assert np.array_equal(_fetch(ex, 1, 0, width, np.float16), by_row.max(axis=0))


def test_layernorm_huge_behind_4_gib(hip_device):
    """slow.rs:12-31: rows of 2^20 floats, with 4 GiB allocated first so that the buffers lie past 32 bit addresses"""
    ballast = DeviceBuffer(hip_device, 4 << 30)
    g = Graph()
    x = g.input([1, 32, 1048576])
    g.output(g.layernorm(x, 2, 1e-6))
    data = np.random.default_rng(0).standard_normal((1, 32, 1048576)).astype(np.float32)
    ex = HipExecutor(hip_device, g, 0)
    ex.upload_input(0, data)
    _run(ex)
    got = _fetch(ex, 0, 0, data.size, np.float32).reshape(data.shape)
    check_outputs(g, 0, [data], cpu_eval_graph(g, 0, [data]), [got], "layernorm_huge", PARITY_RECORDS)
    del ballast


def _check_batches(ex, small, pieces, batch_sizes, out_size, picked, dtype, what):
    """the batch entries `picked` of a batched product, each against the oracle on that entry's operands;
    `pieces[i]` / `batch_sizes[i]`: what input i repeats and how many elements one batch entry of it has"""
    sample = [np.stack([_stretch(piece, z * size, size) for z in picked]) for piece, size in zip(pieces, batch_sizes)]
    sample = [x.reshape(info[1]) for x, info in zip(sample, small.input_info)]
    got = np.stack([_fetch(ex, 0, z * out_size, out_size, dtype) for z in picked]).reshape(small.output_info[0][1])
    oracle_graph = small.graph
    check_outputs(oracle_graph, 0, sample, cpu_eval_graph(oracle_graph, 0, sample), [got], what, PARITY_RECORDS)


class _Small:
    """the same graph over a few batch entries: what the oracle evaluates"""

    def __init__(self, graph):
        self.graph = graph
        plan = HipExecutor(0, graph, 0, plan_only=True)
        self.input_info, self.output_info = plan.input_info, plan.output_info


def _weights_product(batch, rows, k, n, dtype, weights):
    g = Graph()
    a = g.input([batch, rows, k], dtype)
    w = g.constant([1, k, n], weights[None], dtype)
    g.output(g.batched_mat_mul(a, g.broadcast(w, [batch, k, n])))
    return g


def test_f16_product_with_rows_past_2_31_elements(hip_device, block):
    batch, rows, k, n = 2049, 1024, 1024, 64
    weights = (np.random.default_rng(7).standard_normal((k, n)) * 0.05).astype(np.float16)
    ex = HipExecutor(hip_device, _weights_product(batch, rows, k, n, DType.F16, weights), 0)
    _fill_input(ex, 0, block, batch * rows * k)
    _run(ex)
    picked = [0, 1, 1023, 1024, 1025, 2047, 2048]
    _check_batches(ex, _Small(_weights_product(len(picked), rows, k, n, DType.F16, weights)), [block], [rows * k], rows * n,
                   picked, np.float16, "f16 product, 4.3 GB of rows")


def test_f16_batched_product_past_2_31_elements(hip_device, block):
    batch, m, k, n = 16400, 128, 1024, 8

    def build(b):
        g = Graph()
        g.output(g.batched_mat_mul(g.input([b, m, k], DType.F16), g.input([b, k, n], DType.F16)))
        return g

    ex = HipExecutor(hip_device, build(batch), 0)
    _fill_input(ex, 0, block, batch * m * k)
    shifted = np.roll(block, 12345)
    _fill_input(ex, 1, shifted, batch * k * n)
    _run(ex)
    picked = [0, 1, 8191, 8192, 8193, 16398, 16399]
    _check_batches(ex, _Small(build(len(picked))), [block, shifted], [m * k, k * n], m * n, picked, np.float16,
                   "f16 batched product, 16400 entries")


def test_f32_product_with_rows_past_2_31_elements(hip_device, block32):
    batch, rows, k, n = 1025, 2048, 1024, 32
    weights = (np.random.default_rng(8).standard_normal((k, n)) * 0.05).astype(np.float32)
    ex = HipExecutor(hip_device, _weights_product(batch, rows, k, n, DType.F32, weights), 0)
    _fill_input(ex, 0, block32, batch * rows * k)
    _run(ex)
    picked = [0, 1, 511, 512, 513, 1023, 1024]
    _check_batches(ex, _Small(_weights_product(len(picked), rows, k, n, DType.F32, weights)), [block32], [rows * k], rows * n,
                   picked, np.float32, "f32 product, 8.6 GB of rows")


def test_conv_over_an_input_past_2_31_elements(hip_device, block32):
    batch, channels, size, out_channels = 4100, 128, 64, 8
    filters = (np.random.default_rng(9).standard_normal((out_channels, channels, 3, 3)) * 0.05).astype(np.float32)

    def build(b):
        g = Graph()
        x = g.input([b, channels, size, size])
        g.output(g.conv(x, g.constant([out_channels, channels, 3, 3], filters), 1, 1, 1, 1))
        return g

    ex = HipExecutor(hip_device, build(batch), 0)
    _fill_input(ex, 0, block32, batch * channels * size * size)
    _run(ex)
    picked = [0, 1, 4095, 4096, 4097, 4099]
    _check_batches(ex, _Small(build(len(picked))), [block32], [channels * size * size], out_channels * size * size, picked,
                   np.float32, "3x3 conv, 4100 images of 128 x 64 x 64")


def _attention(batch, tokens, width, dtype, causal):
    g = Graph()
    q, k, v = (g.input([batch, tokens, width], dtype) for _ in range(3))
    scores = g.mul(g.batched_mat_mul(q, g.permute(k, [0, 2, 1])), g.scalar(1.0 / np.sqrt(width), dtype))
    if causal:
        mask = np.where(np.tril(np.ones((tokens, tokens), bool)), 0.0, -np.inf).astype(dtype.numpy)
        scores = g.add(scores, g.broadcast(g.constant([1, tokens, tokens], mask[None], dtype), [batch, tokens, tokens]))
    g.output(g.batched_mat_mul(g.softmax(scores, 2), v))
    return g


def test_f16_attention_past_2_31_elements(hip_device, block):
    batch, tokens, width = 32776, 512, 128
    ex = HipExecutor(hip_device, _attention(batch, tokens, width, DType.F16, True), 0)
    assert "attention f16" in ex.step_str(ex.step_count() - 1)
    pieces = [block, np.roll(block, 777), np.roll(block, 31337)]
    for i, piece in enumerate(pieces):
        _fill_input(ex, i, piece, batch * tokens * width)
    _run(ex)
    picked = [0, 1, 16383, 16384, 16385, 32774, 32775]
    _check_batches(ex, _Small(_attention(len(picked), tokens, width, DType.F16, True)), pieces, [tokens * width] * 3,
                   tokens * width, picked, np.float16, "f16 attention, 32776 heads")


def test_f32_attention_with_the_largest_batch(hip_device, block32):
    batch, tokens, width = 65535, 520, 64
    ex = HipExecutor(hip_device, _attention(batch, tokens, width, DType.F32, False), 0)
    assert "attention" in ex.step_str(ex.step_count() - 1)
    pieces = [block32, np.roll(block32, 777), np.roll(block32, 31337)]
    for i, piece in enumerate(pieces):
        _fill_input(ex, i, piece, batch * tokens * width)
    _run(ex)
    picked = [0, 1, 32767, 32768, 32769, 65533, 65534]
    _check_batches(ex, _Small(_attention(len(picked), tokens, width, DType.F32, False)), pieces, [tokens * width] * 3,
                   tokens * width, picked, np.float32, "f32 attention, 65535 heads")
