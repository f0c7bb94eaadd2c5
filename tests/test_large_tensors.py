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


def _fill_input(ex, index, block, dtype, count):
    """input `index` := the block's bytes, read as `dtype`, repeated over `count` elements"""
    piece = block.view(dtype)
    done = 0
    while done < count:
        step = min(piece.size, count - done)
        check(lib.knhip_memcpy_h2d(ex.device, c_void_p(ex.input_ptr(index) + done * piece.itemsize), piece.ctypes.data, step * piece.itemsize))
        done += step
    return piece


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
    piece = _fill_input(ex, 0, block, np.uint8, n)
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
    piece = _fill_input(ex, 0, block, np.uint8, rows * cols)
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
    piece = _fill_input(ex, 0, block, np.uint8, n)
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
    _fill_input(ex, 0, block, np.float16, rows * width)
    _run(ex)
    picked = _row_samples(rows)
    got = np.stack([_fetch(ex, 0, r * width, width, np.float16) for r in picked])
    sample = np.ascontiguousarray(block.reshape(-1, width)[[r % (BLOCK // width) for r in picked]])
    small = Graph()
    sx = small.input([len(picked), width], DType.F16)
    small.output(small.softmax(sx, 1))
    check_outputs(small, 0, [sample], cpu_eval_graph(small, 0, [sample]), [got], "softmax rows of a 4 GiB tensor", PARITY_RECORDS)


def test_reduce_past_2_31_elements(hip_device, block):
    rows, width = (1 << 19) + 1, BLOCK_WIDTH
    g = Graph()
    x = g.input([rows, width], DType.F16)
    g.output(g.reduce(x, [1], ReduceOp.SUM))
    g.output(g.reduce(x, [0], ReduceOp.MAX))
    ex = HipExecutor(hip_device, g, 0)
    _fill_input(ex, 0, block, np.float16, rows * width)
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
