"""The parity rules themselves (oracle/parity.py) and the f64 evaluator they lean on (oracle/f64_eval.py).

* The f64 evaluator is a third implementation of the graph semantics; here it meets the oracle on every graph
  case of the suite, so a mistake in either shows up without a GPU.
* A correct result computed in another summation order passes the rules, and planted defects of the size real
  kernel bugs have (a dropped term, a swapped index, one wrong element, a missing bias) fail them.
"""
import numpy as np
import pytest

from cases_graphs import CASES
from kyanite_amd import DType, Graph
from oracle import cpu_eval_graph
from oracle.f64_eval import Unsupported, eval_graph_f64
from oracle.parity import (F16_MAX_REL, F32_MAX_REL, SMALL_FLOOR, accumulation_length, check_outputs, is_exact_graph,
                           k_floor, rel_error)


@pytest.mark.parametrize("name", list(CASES))
def test_f64_evaluator_meets_oracle(name):
    graph, batch, inputs, _ = CASES[name]()
    oracle_outputs = cpu_eval_graph(graph, batch, inputs)
    try:
        exact = eval_graph_f64(graph, batch, inputs, storage_rounding=True)
    except Unsupported as why:
        pytest.skip(f"not evaluable in f64: {why}")
    assert len(exact) == len(oracle_outputs)
    for t, e in zip(exact, oracle_outputs):
        assert list(t.shape) == list(e.shape)
        if e.dtype.kind != "f":
            assert np.array_equal(t, e)
            continue
        # Same roundings of stored values on both sides, exact arithmetic inside each operation on one of them: what
        # is left is the oracle's f32 arithmetic, and values that land on the neighbouring f16 / f32 number and are
        # amplified by later cancellations. A difference in MEANING (another axis, formula or operand) is of the
        # order of the tensor's rms.
        err = rel_error(t, e, 0.1)
        bar = 5e-2 if e.dtype == np.float16 else 1e-3
        assert err <= bar, f"{name}: oracle is {err:.3e} from the f64 evaluation"


def _matmul_graph(m, k, n, seed, bias=False):
    rng = np.random.default_rng(seed)
    g = Graph()
    x = g.input([m, k])
    w = rng.standard_normal((k, n)).astype(np.float32)
    y = g.mat_mul(x, g.constant([k, n], w))
    b = None
    if bias:
        b = rng.standard_normal((1, n)).astype(np.float32)
        y = g.add(y, g.constant([1, n], b))
    g.output(y)
    return g, rng.standard_normal((m, k)).astype(np.float32), w, b


def test_reordered_sum_passes_and_defects_fail():
    m, k, n = 48, 4096, 40
    g, x, w, b = _matmul_graph(m, k, n, 1, bias=True)
    oracle = cpu_eval_graph(g, 0, [x])
    # the same product summed in blocks of 64, as a tiled kernel does
    blocks = [x[:, i:i + 64] @ w[i:i + 64] for i in range(0, k, 64)]
    tiled = (np.sum(np.stack(blocks), axis=0, dtype=np.float32) + b).astype(np.float32)
    records = []
    check_outputs(g, 0, [x], oracle, [tiled], "tiled", records)
    assert records[0]["rule"] in ("direct", "accumulated")

    def fails(candidate):
        with pytest.raises(AssertionError):
            check_outputs(g, 0, [x], oracle, [candidate.astype(np.float32)], "defect")

    fails(tiled - x[:, -1:] * w[-1:, :])                 # last term of every sum dropped
    fails(tiled - b)                                      # bias forgotten
    wrong = tiled.copy()
    wrong[7, 3] = tiled[7, 4]
    fails(wrong)                                          # one element read from its neighbour
    fails(tiled * np.float32(1.001))                      # a scale off by a thousandth
    shifted = ((x[:, 1:] @ w[:-1]) + b)
    fails(shifted)                                        # operand index off by one


def test_small_elements_need_the_f64_rule_not_a_wide_floor():
    """An output far below its tensor's rms that is wrong by a tenth of its own size fails every rule."""
    m, k, n = 32, 1024, 32
    g, x, w, _ = _matmul_graph(m, k, n, 2)
    oracle = cpu_eval_graph(g, 0, [x])[0]
    exact = eval_graph_f64(g, 0, [x])[0]
    i, j = np.unravel_index(np.argmin(np.abs(exact)), exact.shape)
    rms = float(np.sqrt(np.mean(exact * exact)))
    assert abs(exact[i, j]) < 0.01 * rms
    wrong = oracle.copy()
    wrong[i, j] += np.float32(0.02 * rms)
    with pytest.raises(AssertionError):
        check_outputs(g, 0, [x], [oracle], [wrong], "small element")


def test_exact_class():
    g = Graph()
    x = g.input([4, 6])
    g.output(g.add(g.permute(x, [1, 0]), g.constant([6, 4], np.arange(24, dtype=np.float32))))
    assert is_exact_graph(g) and accumulation_length(g, 0) == 0
    a = np.linspace(-1, 1, 24, dtype=np.float32).reshape(4, 6)
    oracle = cpu_eval_graph(g, 0, [a])
    records = []
    check_outputs(g, 0, [a], oracle, [oracle[0].copy()], "exact", records)
    assert records[0]["rule"] == "exact"
    off = oracle[0].copy()
    off[2, 1] = np.nextafter(off[2, 1], np.float32(10))
    with pytest.raises(AssertionError):
        check_outputs(g, 0, [a], oracle, [off], "one ulp")

    h = Graph()
    y = h.input([4, 6])
    h.output(h.unary(8, y))  # tanh
    assert not is_exact_graph(h)


def test_f16_graph_classes():
    g = Graph()
    x = g.input([16, 256], DType.F16)
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((256, 24)) * 0.1).astype(np.float16)
    g.output(g.mat_mul(x, g.constant([256, 24], w, DType.F16)))
    a = rng.standard_normal((16, 256)).astype(np.float16)
    oracle = cpu_eval_graph(g, 0, [a])
    assert accumulation_length(g, 0) == 256
    blocked = sum((a[:, i:i + 32].astype(np.float32) @ w[i:i + 32].astype(np.float32)) for i in range(0, 256, 32))
    check_outputs(g, 0, [a], oracle, [blocked.astype(np.float16)], "f16 blocked")
    with pytest.raises(AssertionError):
        check_outputs(g, 0, [a], oracle, [(blocked * 1.05).astype(np.float16)], "f16 scaled")
