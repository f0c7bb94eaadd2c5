"""Differential test harness in the style of kn-cuda-eval/tests/root/runner.rs:10-55.

`check_cpu` runs the oracle (checked against expected values when the reference's test holds them) on the
unoptimized and the optimized graph, and plans + compiles both graphs without a device.
`check_gpu` runs the HIP executor on both graphs and compares against expected-or-oracle.
"""
import numpy as np

from kyanite_amd import HipExecutor, optimize_graph
from oracle import cpu_eval_graph

# kn-cuda-eval/src/tester.rs:28-29: a float only mismatches when BOTH differences reach the tolerance
TOLERANCE_ABS_DIFF = 0.001
TOLERANCE_REL_DIFF = 0.001

# The tighter bars this project states for its own GPU path against the oracle live in oracle/parity.py:
# bit-exact for data movement and IEEE-fixed arithmetic, 1e-4 (f32) / 2e-2 (f16) with a floor of 1e-3 rms for
# everything else, and for sums of K terms an f64-referenced rule that asks the GPU result to be no further
# from the exact value than the oracle is.
from oracle.parity import F16_MAX_REL, F32_MAX_REL, SMALL_FLOOR, check_outputs, rel_error

# one dict per compared output of every GPU check of the session (conftest.py writes them out at the end)
PARITY_RECORDS = []


def assert_tensors_match(expected, actual, what=""):
    """tester.rs:31-120: exact for ints and bools, abs-and-rel tolerance for floats, NaN must match NaN."""
    assert len(expected) == len(actual), f"{what}: wrong output count {len(actual)}, expected {len(expected)}"
    for i, (e, a) in enumerate(zip(expected, actual)):
        e = np.asarray(e)
        a = np.asarray(a)
        assert list(e.shape) == list(a.shape), f"{what}: output {i} shape {a.shape}, expected {e.shape}"
        assert e.dtype == a.dtype, f"{what}: output {i} dtype {a.dtype}, expected {e.dtype}"
        if e.dtype.kind in "fc":
            e64, a64 = e.astype(np.float64), a.astype(np.float64)
            nan_mismatch = np.isnan(e64) != np.isnan(a64)
            with np.errstate(invalid="ignore", divide="ignore"):
                same = (e64 == a64) | np.isnan(e64) | np.isnan(a64)
                abs_diff = np.where(same, 0.0, np.abs(e64 - a64))
                rel_diff = np.where(same, 0.0, abs_diff / np.abs(e64))
            tol_abs, tol_rel = (F16_MAX_REL, F16_MAX_REL) if e.dtype == np.float16 else (TOLERANCE_ABS_DIFF, TOLERANCE_REL_DIFF)
            bad = ((abs_diff >= tol_abs) & (rel_diff >= tol_rel)) | nan_mismatch
            if bad.any():
                idx = np.argwhere(bad)[:8]
                lines = [f"  {tuple(j)}: expected {e[tuple(j)]}, got {a[tuple(j)]}" for j in idx]
                raise AssertionError(f"{what}: output {i} mismatch in {bad.sum()}/{bad.size} values:\n" + "\n".join(lines))
        else:
            if not np.array_equal(e, a):
                bad = e != a
                idx = np.argwhere(bad)[:8]
                lines = [f"  {tuple(j)}: expected {e[tuple(j)]}, got {a[tuple(j)]}" for j in idx]
                raise AssertionError(f"{what}: output {i} mismatch in {bad.sum()}/{bad.size} values:\n" + "\n".join(lines))


# Golden vectors were written by another f32 implementation (the exporter's runtime), so both sides of a comparison
# with them carry rounding noise of their own; the reference accepts abs 1e-3 and rel 1e-3 for them.
GOLDEN_FLOOR = 0.1


def assert_close(expected, actual, what="", max_rel=F32_MAX_REL, floor=GOLDEN_FLOOR):
    """Against vectors that come without an oracle run (golden files): bit-exact for ints / bools, `max_rel` with
    `floor` (a fraction of the tensor's rms) for floats."""
    assert len(expected) == len(actual)
    for i, (e, a) in enumerate(zip(expected, actual)):
        assert list(e.shape) == list(a.shape) and e.dtype == a.dtype, f"{what}: output {i} shape/dtype mismatch"
        if e.dtype.kind == "f":
            err = rel_error(e, a, floor)
            bar = F16_MAX_REL if e.dtype == np.float16 else max_rel
            assert err <= bar, f"{what}: output {i} max relative error {err:.3e} exceeds {bar:.1e}"
        else:
            assert np.array_equal(e, a), f"{what}: output {i} differs (exact match required for {e.dtype})"


def check_cpu(graph, batch_size, inputs, expected=None):
    """CPU half of `test_all`: oracle vs expected on the graph and on its optimized form; both must also plan
    and compile for the GPU (no device needed)."""
    cpu_outputs = cpu_eval_graph(graph, batch_size, inputs)
    if expected is not None:
        assert_tensors_match(expected, cpu_outputs, "oracle, unoptimized")
    reference = expected if expected is not None else cpu_outputs
    optimized = optimize_graph(graph)
    cpu_optimized = cpu_eval_graph(optimized, batch_size, inputs)
    assert_tensors_match(reference, cpu_optimized, "oracle, optimized")
    HipExecutor(0, graph, batch_size, plan_only=True)
    HipExecutor(0, optimized, batch_size, plan_only=True)
    return cpu_outputs


def check_gpu(device, graph, batch_size, inputs, expected=None, what=""):
    """GPU half of `test_all`: the HIP executor on the graph and on its optimized form against
    expected-or-oracle with the reference's tolerance, and against the oracle on the same graph with this
    project's own rules (oracle/parity.py)."""
    cpu_outputs = cpu_eval_graph(graph, batch_size, inputs)
    reference = expected if expected is not None else cpu_outputs
    results = []
    for name, g in (("unoptimized", graph), ("optimized", optimize_graph(graph))):
        cpu_same_graph = cpu_outputs if name == "unoptimized" else cpu_eval_graph(g, batch_size, inputs)
        ex = HipExecutor(device, g, batch_size)
        # a plan of a few tiny steps runs as ONE kernel: then the steps are checked launched one by one as well, and
        # so is the path of callers that write the inputs on the device themselves (run_async on arena addresses)
        executors = [(name, ex)]
        if ex.fused_source():
            executors.append((name + ", step by step", HipExecutor(device, g, batch_size, step_by_step=True)))
        for label, e in executors:
            gpu_outputs = e.evaluate(inputs)
            assert_tensors_match(reference, gpu_outputs, f"gpu, {label}")
            check_outputs(g, batch_size, inputs, cpu_same_graph, gpu_outputs, f"{what} {label}".strip(), PARITY_RECORDS)
            # a second evaluation must give the same answer (buffers are reused between calls)
            again = e.evaluate(inputs)
            for x, y in zip(gpu_outputs, again):
                assert np.array_equal(x, y, equal_nan=True), f"gpu, {label}: second evaluation differs"
        results.append(gpu_outputs)
    return results[0]


def linspace_tensor(*shape):
    n = int(np.prod(shape)) if shape else 1
    return np.linspace(-1.0, 1.0, n, dtype=np.float64).astype(np.float32).reshape(shape)


def linspace_vec(n):
    return np.linspace(-1.0, 1.0, n, dtype=np.float64).astype(np.float32)


def range_vec(n):
    return np.arange(n, dtype=np.float32)


def rng_tensor(rng, *shape):
    """Uniform [0, 1) like `rng.gen::<f32>()`; the reference's exact stream is not reproducible without Rust,
    and every test that uses it compares against the CPU path, so any seeded stream keeps the intent."""
    return rng.random(shape, dtype=np.float32)
