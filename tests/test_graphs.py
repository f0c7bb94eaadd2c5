"""The reference's graph tests (kn-cuda-eval/tests/root/graphs.rs), CPU half and GPU half.

CPU (not gpu): the oracle against the expected values the reference holds, on the unoptimized and the optimized
graph, and both graphs must plan and compile for gfx950. GPU: the HIP executor against expected-or-oracle.
"""
import pytest

from cases_graphs import CASES
from runner import F32_MAX_REL, check_cpu, check_gpu

# Cases whose f32 rounding differences compound over several chained contractions with cancelling terms get a
# wider (still stated) bound against the oracle; everything else has to meet F32_MAX_REL.
MAX_REL_OVERRIDES = {
}


@pytest.mark.parametrize("name", list(CASES))
def test_cpu(name):
    graph, batch, inputs, expected = CASES[name]()
    check_cpu(graph, batch, inputs, expected)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(CASES))
def test_gpu(name, hip_device):
    graph, batch, inputs, expected = CASES[name]()
    print(f"case {name} batch {batch}", flush=True)
    check_gpu(hip_device, graph, batch, inputs, expected, MAX_REL_OVERRIDES.get(name, F32_MAX_REL))
