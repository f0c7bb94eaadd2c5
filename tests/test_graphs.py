"""The reference's graph tests (kn-cuda-eval/tests/root/graphs.rs), CPU half and GPU half.

CPU (not gpu): the oracle against the expected values the reference holds, on the unoptimized and the optimized
graph, and both graphs must plan and compile for gfx950. GPU: the HIP executor against expected-or-oracle.
"""
import pytest

from cases_graphs import CASES
from runner import check_cpu, check_gpu

@pytest.mark.parametrize("name", list(CASES))
def test_cpu(name):
    graph, batch, inputs, expected = CASES[name]()
    check_cpu(graph, batch, inputs, expected)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(CASES))
def test_gpu(name, hip_device):
    graph, batch, inputs, expected = CASES[name]()
    print(f"case {name} batch {batch}", flush=True)
    check_gpu(hip_device, graph, batch, inputs, expected, what=name)
