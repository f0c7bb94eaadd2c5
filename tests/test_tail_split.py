"""The in-launch K split of the direct matmul kernel (the tiles of a sparse last round of workgroups are shared by
2..16 workgroups that exchange f32 partial tiles and count themselves in on a per-tile counter) in every
instantiation the launch plan picks: f32 on 64 x 64 and 128 x 128 tiles, f16 on 64 x 64, 128 x 64, 256 x 192 and
256 x 256 tiles (with the f16 cost model a sparse last round of 128 x 128 or 256 x 128 tiles never comes out cheapest:
a larger tile that fits one round does), splits of 2, 3, 4 and 8, epilogues (bias, residual, relu), ragged tile rows
and grouped launches, and the grouped f32 launches of a handful of tiles, all of which are shared. The GPU multiplies the whole product, twice (the second run finds the counters as the first left them); the
oracle evaluates the same graph on a sample of the rows of the left operand that reaches every tile row of every
workgroup tile, and those rows of the GPU result are compared with it."""
import numpy as np
import pytest

from kyanite_amd import DType, Graph, HipExecutor
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

# dtype, m, n, k, (bias, residual, relu), number of products that share the left operand, expected in the plan
CASES = [
    (DType.F32, 33, 33280, 1536, (True, False, False), 1, "direct 64x64 bk32 head=512 tail_split=3x512"),
    (DType.F32, 250, 33280, 1024, (True, True, True), 1, "direct 128x128 bk32 head=512 tail_split=2x512"),
    (DType.F32, 256, 2816, 1024, (False, False, False), 3, "x3 grouped [direct 64x64 bk32 head=512 tail_split=2x512"),
    (DType.F32, 512, 5632, 2048, (False, False, False), 3, "x3 grouped [direct 128x128 bk32 head=512 tail_split=4x512"),
    (DType.F16, 33, 33280, 4096, (False, False, False), 1, "direct 64x64 bk64 head=512 tail_split=8x512"),
    (DType.F16, 256, 8320, 2048, (True, False, True), 1, "direct 128x64 bk64 head=256 tail_split=4x512"),
    (DType.F16, 256, 10368, 2048, (False, True, False), 1, "direct 128x64 bk64 head=256 tail_split=3x704"),
    (DType.F16, 300, 33088, 1024, (True, True, False), 1, "direct 256x192 bk64 head=256 tail_split=2x512"),
    (DType.F16, 768, 24768, 2048, (False, True, True), 1, "direct 256x256 bk64 head=256 tail_split=4x512"),
    (DType.F16, 768, 24768, 1536, (True, False, False), 1, "direct 256x256 bk64 head=256 tail_split=3x512"),
    (DType.F16, 300, 2688, 1536, (False, False, False), 3, "x3 grouped [direct 64x64 bk64 head=512 tail_split=3x512"),
    (DType.F16, 300, 11008, 1024, (False, False, False), 3, "x3 grouped [direct 256x192 bk64 head=256 tail_split=2x512"),
    (DType.F16, 1024, 6528, 2048, (False, False, False), 3, "x3 grouped [direct 256x256 bk64 head=256 tail_split=4x512"),
    # a handful of tiles in a grouped f32 launch: every tile shared (head = 0)
    (DType.F32, 154, 320, 768, (False, False, False), 2, "x2 grouped [direct 64x64 bk32 head=0 tail_split=6x128"),
    (DType.F32, 100, 200, 2144, (False, False, False), 3, "x3 grouped [direct 128x128 bk32 head=0 tail_split=14x160"),
]


def _build(dtype, m, n, k, epilogue, products, weights):
    """`weights`: constant [n, k] right operands for a grouped launch, else the right operand is an input."""
    bias, residual, relu = epilogue
    g = Graph()
    x = g.input([m, k], dtype)
    if products > 1:
        for w in weights:
            g.output(g.linear(x, g.constant([n, k], w, dtype)))
        return g
    y = g.linear(x, g.input([n, k], dtype))
    if bias:
        y = g.add(y, g.input([1, n], dtype))
    if residual:
        y = g.add(g.input([m, n], dtype), y)
    if relu:
        y = g.relu(y)
    g.output(y)
    return g


def _sample_rows(m):
    """a few rows of every 32 row MFMA tile row: each wave of each workgroup tile stores some of them"""
    rows = sorted({r for base in range(0, m, 32) for r in (base, base + 13, base + 31) if r < m})
    return np.array(rows)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0].name}-{c[1]}x{c[2]}x{c[3]}-x{c[5]}-{c[6].split('direct ')[1].split(' ')[0]}")
def test_tail_split(case, hip_device):
    dtype, m, n, k, epilogue, products, expected_plan = case
    np_dtype = np.float16 if dtype == DType.F16 else np.float32
    scale = 0.2 if dtype == DType.F16 else 1.0
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    x = (rng.standard_normal((m, k)) * scale).astype(np_dtype)
    weights = [(rng.standard_normal((n, k)) * scale).astype(np_dtype) for _ in range(products)]
    inputs = [x]
    if products == 1:
        inputs.append(weights[0])
        if epilogue[0]:
            inputs.append(rng.standard_normal((1, n)).astype(np_dtype))
        if epilogue[1]:
            inputs.append(rng.standard_normal((m, n)).astype(np_dtype))
    graph = _build(dtype, m, n, k, epilogue, products, weights)
    print(f"tail split {dtype.name} {m}x{n}x{k} x{products} {epilogue}", flush=True)
    ex = HipExecutor(hip_device, graph, 0)
    plans = [ex.step_str(i) for i in range(ex.step_count())]
    assert any(expected_plan in p for p in plans), f"the plan no longer takes the path under test: {plans}"

    rows = _sample_rows(m)
    sampled_inputs = [x[rows]] + [a[rows] if a.shape[0] == m and a.ndim == 2 and a.shape[1] == n else a for a in inputs[1:]]
    sampled_graph = _build(dtype, len(rows), n, k, epilogue, products, weights)
    expected = cpu_eval_graph(sampled_graph, 0, sampled_inputs)
    for run in range(2):
        got = ex.evaluate(inputs)
        check_outputs(sampled_graph, 0, sampled_inputs, expected, [o[rows] for o in got],
                      f"tail split {case[:4]} x{products} run {run}", PARITY_RECORDS)
