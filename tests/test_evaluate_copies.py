"""`evaluate` moves tensors of more than 2 MiB in chunks of a quarter of the tensor, 2 MiB at least and 8 MiB at most
(host copy of one chunk while the copy engine moves another)
and spreads big host copies over threads: results must not depend on where the chunk boundaries fall
(kn-cuda-eval/src/executor.rs:117-195 is the path; the reference copies every tensor in one piece)."""
import numpy as np
import pytest

from kyanite_amd import DType, Graph, HipExecutor, KnError
from oracle import cpu_eval_graph

CHUNK, LEAST = 8 << 20, 2 << 20


@pytest.mark.gpu
@pytest.mark.parametrize("elements", [CHUNK // 4 - 1, CHUNK // 4, CHUNK // 4 + 1, 3 * (CHUNK // 4) + 12345, 1,
                                      LEAST // 4, LEAST // 4 + 1, LEAST + 77, 4 * CHUNK // 4 + 3, 5 * (CHUNK // 4) + 1])
def test_tensors_around_the_chunk_size_arrive_whole(elements, hip_device):
    print(f"evaluate with {elements} f32 elements per tensor", flush=True)
    g = Graph()
    x, k = g.input([elements]), g.input([elements], DType.I32)
    g.output_all([g.add(x, g.scalar(1.0)), k, g.add(k, k)])
    rng = np.random.default_rng(elements)
    inputs = [rng.standard_normal(elements).astype(np.float32), rng.integers(-2 ** 31, 2 ** 31 - 1, elements, dtype=np.int32)]
    ex = HipExecutor(hip_device, g, 0)
    expected = cpu_eval_graph(g, 0, inputs)
    got = ex.evaluate(inputs)
    for e, a in zip(expected, got):
        assert np.array_equal(e, a)
    # a second evaluation into the caller's arrays, with other inputs: nothing of the first one may survive
    inputs2 = [inputs[0][::-1].copy(), inputs[1][::-1].copy()]
    out = [np.full_like(a, 7) for a in got]
    assert ex.evaluate(inputs2, out=out)[0] is out[0]
    for e, a in zip(cpu_eval_graph(g, 0, inputs2), out):
        assert np.array_equal(e, a)


def test_out_arrays_are_checked():
    g = Graph()
    g.output(g.add(g.input([4, 4]), g.scalar(1.0)))
    ex = HipExecutor(0, g, 0, plan_only=True)
    x = [np.zeros((4, 4), np.float32)]
    for bad in ([np.zeros((4, 4), np.float64)], [np.zeros((4, 5), np.float32)], [np.zeros((8, 4), np.float32)[::2]], []):
        with pytest.raises(KnError):
            ex.evaluate(x, out=bad)
