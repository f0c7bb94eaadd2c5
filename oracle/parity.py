"""ORACLE - test infrastructure only (tests, the smoke check and the benchmark's parity leg).

The bars a GPU result has to meet against the CPU oracle (`cpu_eval_graph`), one rule per class of graph:

exact        graphs that only move data or do arithmetic that IEEE fixes bit for bit (layout operations, gather,
             concat, casts, integer / bool arithmetic, float + - * min max abs neg): every output bit-equal.
direct       every other float output:  max |a - e| / max(|e|, 1e-3 * rms(e))  <=  1e-4 (f32), 2e-2 (f16).
             This is the stated bar with the small floor that sums crossing zero need
             (kn-cuda-eval/src/tester.rs:264-281 has an absolute floor of 1e-3 for the same reason).
accumulated  only for graphs that sum K terms per output element (matmul, conv, sum / mean / prod reductions,
             layernorm statistics), and only when `direct` is not met. Two f32 evaluations of a K-term sum that
             differ in the ORDER of the additions differ by rounding noise of about u * sqrt(K) * rms per element
             (u = 2^-24), whatever either of them does, and f16 graphs round every intermediate value to 11 bits;
             for elements far below the tensor's rms that noise is not small relative to the element, and it is
             as much the oracle's as the kernel's. Such an output passes when both hold:
               (1) against an f64 evaluation t of the same graph (f64_eval.py, no intermediate rounding), the GPU
                   result is no further from the exact value than the oracle is, in the largest and in the mean
                   deviation:  max |gpu - t| <= 2 max |oracle - t| + tiny rms(t)  and
                   rms(gpu - t) <= 2 rms(oracle - t) + tiny rms(t),  tiny = 16 u (f32) or one f16 ulp.
                   (Deviations are compared as they are, not divided by |t|: the noise of an element depends on
                   the size of the terms that were summed, not on the size of what is left of them.)
               (2) gpu and oracle agree within the bar once the floor is raised to the noise level (`k_floor`):
                   a wrong index or a dropped term shows up as an error of the order of the rms itself and fails
                   this however large K is. Waived only when the oracle itself is further than half the bar from
                   the f64 result under that same floor (an ill-conditioned graph: a difference of nearly equal
                   values magnified by a division), where (1) alone decides.
NaN and infinities must agree exactly under every rule.
"""
import math

import numpy as np

from .f64_eval import DType, OpKind, ReduceOp, UnaryOp, BinaryOp, Unsupported, eval_graph_f64

F32_MAX_REL = 1e-4
F16_MAX_REL = 2e-2
SMALL_FLOOR = 1e-3
U32 = 2.0 ** -24  # unit roundoff of f32
U16 = 2.0 ** -11  # unit roundoff of f16
TINY_F32 = 16 * U32
TINY_F16 = 2 * U16


def _float(dtype):
    return int(dtype) in (DType.F32, DType.F64, DType.F16)


def accumulation_length(graph, batch_size):
    """Longest sum any single operation of the graph forms per output element (0: the graph sums nothing)."""
    longest = 0
    for v in graph.values():
        info = graph[v]
        if not _float(info.dtype):
            continue
        if info.op == OpKind.MATMUL:
            k = graph[info.operands[0]].shape[-1].eval(batch_size)
        elif info.op == OpKind.CONV:
            f = graph[info.operands[1]].shape
            k = f[1].eval(batch_size) * f[2].eval(batch_size) * f[3].eval(batch_size)
        elif info.op == OpKind.REDUCE and info.sub_op in (ReduceOp.SUM, ReduceOp.MEAN, ReduceOp.PROD):
            src = graph[info.operands[0]].shape
            k = int(np.prod([src[a].eval(batch_size) for a in info.axes])) if info.axes else 1
        elif info.op == OpKind.LAYERNORM:
            # mean and variance are sums too, but their rounding error reaches the output divided by the row
            # length: eligible for the rule, without raising the noise floor
            k = 1
        else:
            continue
        longest = max(longest, int(k))
    return longest


_EXACT_UNARY = (UnaryOp.ABS, UnaryOp.NEG, UnaryOp.VALUE_CAST, UnaryOp.BIT_CAST)
_EXACT_BINARY = (BinaryOp.ADD, BinaryOp.SUB, BinaryOp.MUL, BinaryOp.MIN, BinaryOp.MAX)


def is_exact_graph(graph):
    """True when IEEE arithmetic fixes every output bit: no operation whose float result depends on how it is
    implemented (transcendentals, division, roots, sums of many terms)."""
    for v in graph.values():
        info = graph[v]
        if not _float(info.dtype):
            continue
        if info.op in (OpKind.MATMUL, OpKind.CONV, OpKind.SOFTMAX, OpKind.LAYERNORM):
            return False
        if info.op == OpKind.REDUCE and info.sub_op not in (ReduceOp.MAX, ReduceOp.MIN):
            return False
        if info.op == OpKind.UNARY and info.sub_op not in _EXACT_UNARY:
            return False
        if info.op == OpKind.BINARY and info.sub_op not in _EXACT_BINARY:
            return False
    return True


def k_floor(k, f16):
    """Floor (as a fraction of the tensor's rms) at which two correct evaluations that differ only in rounding
    still agree within the bar.
    f32: two orders of a K-term sum differ by about u * sqrt(K) * rms (one standard deviation); 8 of those.
    f16: every stored value is rounded to f16, and an f32 result that sits near a rounding boundary lands on either
    neighbour depending on summation order: one f16 ulp (2^-10) of an intermediate value, which may be several
    times larger than what remains after later additions. One ulp of a value 4 rms large stays inside the bar."""
    if f16:
        return max(SMALL_FLOOR, 4 * 2 * U16 / F16_MAX_REL)
    return max(SMALL_FLOOR, 8 * U32 * math.sqrt(k) / F32_MAX_REL)


def rel_error(expected, actual, floor_fraction):
    """max |a - e| / max(|e|, floor_fraction * rms(e)) over the elements where e is finite; NaN and infinities of e
    must be matched exactly by a."""
    e = np.asarray(expected, dtype=np.float64).reshape(-1)
    a = np.asarray(actual, dtype=np.float64).reshape(-1)
    special = ~np.isfinite(e)
    if special.any():
        assert np.array_equal(e[special], a[special], equal_nan=True), "non-finite values differ"
        e, a = e[~special], a[~special]
    if e.size == 0:
        return 0.0
    assert np.isfinite(a).all(), "actual holds non-finite values where expected is finite"
    floor = floor_fraction * math.sqrt(float(np.mean(e * e)))
    return float(np.max(np.abs(a - e) / np.maximum(np.abs(e), max(floor, 1e-300))))


def floor_needed(expected, actual, bar):
    """The smallest floor, as a fraction of rms(expected), under which `rel_error(expected, actual, floor) <= bar`:
    0 when every element is within the bar relative to itself, else the largest |a - e| / bar among the elements that
    are not, over the rms. It says how far below the tensor's rms an element has to lie before the two sides stop
    agreeing to `bar` of it."""
    e = np.asarray(expected, dtype=np.float64).reshape(-1)
    a = np.asarray(actual, dtype=np.float64).reshape(-1)
    keep = np.isfinite(e) & np.isfinite(a)
    e, a = e[keep], a[keep]
    if e.size == 0:
        return 0.0
    d = np.abs(a - e)
    outside = d > bar * np.abs(e)
    if not outside.any():
        return 0.0
    rms = max(math.sqrt(float(np.mean(e * e))), 1e-300)
    return float(d[outside].max() / bar / rms)


def _deviation(exact, x, keep):
    """(largest, root mean square) deviation of x from the exact values, as fractions of rms(exact)."""
    t = np.asarray(exact, dtype=np.float64).reshape(-1)
    x = np.asarray(x, dtype=np.float64).reshape(-1)
    keep = keep & np.isfinite(t)
    if not keep.any():
        return 0.0, 0.0
    t, x = t[keep], x[keep]
    scale = max(math.sqrt(float(np.mean(t * t))), 1e-300)
    d = np.abs(x - t)
    return float(d.max() / scale), float(math.sqrt(float(np.mean(d * d))) / scale)


def _bits_equal(e, a):
    e, a = np.ascontiguousarray(e), np.ascontiguousarray(a)
    if e.dtype.kind == "f":
        both_nan = np.isnan(e) & np.isnan(a)
        view = {2: np.uint16, 4: np.uint32, 8: np.uint64}[e.dtype.itemsize]
        return bool(np.all((e.view(view) == a.view(view)) | both_nan))
    return bool(np.array_equal(e, a))


def check_outputs(graph, batch_size, inputs, oracle_outputs, gpu_outputs, what="", records=None, exact_outputs=None):
    """Assert the rules of this module for every output; appends one dict per output to `records`.
    `exact_outputs` may carry the f64 evaluation when the caller already has it."""
    assert len(oracle_outputs) == len(gpu_outputs), f"{what}: {len(gpu_outputs)} outputs, expected {len(oracle_outputs)}"
    exact_graph = is_exact_graph(graph)
    k = accumulation_length(graph, batch_size)
    for i, (e, a) in enumerate(zip(oracle_outputs, gpu_outputs)):
        e, a = np.asarray(e), np.asarray(a)
        assert list(e.shape) == list(a.shape) and e.dtype == a.dtype, \
            f"{what}: output {i} is {a.dtype}{list(a.shape)}, expected {e.dtype}{list(e.shape)}"
        record = {"what": what, "output": i, "dtype": str(e.dtype), "elements": int(e.size), "k": k}
        if records is not None:
            records.append(record)
        if e.dtype.kind != "f" or exact_graph:
            record["rule"] = "exact"
            assert _bits_equal(e, a), f"{what}: output {i} differs (bit-exact match required for this graph)"
            continue
        f16 = e.dtype == np.float16
        bar = F16_MAX_REL if f16 else F32_MAX_REL
        err = rel_error(e, a, SMALL_FLOOR)
        record["err"] = err
        record["floor_needed"] = floor_needed(e, a, bar)
        if err <= bar:
            record["rule"] = "direct"
            continue
        assert k > 0, f"{what}: output {i} max relative error {err:.3e} exceeds {bar:.1e} (floor {SMALL_FLOOR} rms)"
        if exact_outputs is None:
            try:
                exact_outputs = eval_graph_f64(graph, batch_size, inputs)
            except Unsupported as why:
                raise AssertionError(f"{what}: output {i} needs the f64 evaluation to pass ({err:.3e} > {bar:.1e}) "
                                     f"and the graph cannot be evaluated in f64: {why}")
        finite = np.isfinite(e.astype(np.float64).reshape(-1)) & np.isfinite(a.astype(np.float64).reshape(-1))
        gpu_max, gpu_rms = _deviation(exact_outputs[i], a, finite)
        oracle_max, oracle_rms = _deviation(exact_outputs[i], e, finite)
        floor = k_floor(k, f16)
        err_k = rel_error(e, a, floor)
        oracle_k = rel_error(np.where(np.isfinite(exact_outputs[i]), exact_outputs[i], e.astype(np.float64)), e, floor)
        record.update(rule="accumulated", floor_k=floor, err_k=err_k, oracle_err_k=oracle_k, gpu_max=gpu_max, gpu_rms=gpu_rms,
                      oracle_max=oracle_max, oracle_rms=oracle_rms, rule2_waived=bool(err_k > bar))
        tiny = TINY_F16 if f16 else TINY_F32
        assert gpu_max <= 2 * oracle_max + tiny and gpu_rms <= 2 * oracle_rms + tiny, \
            (f"{what}: output {i} is further from the f64 result (max {gpu_max:.3e}, rms {gpu_rms:.3e} of the tensor's "
             f"rms) than twice the oracle (max {oracle_max:.3e}, rms {oracle_rms:.3e}) plus {tiny:.1e}")
        assert err_k <= bar or oracle_k > bar / 2, \
            (f"{what}: output {i} max relative error {err_k:.3e} exceeds {bar:.1e} even with the floor for sums of "
             f"{k} terms ({floor:.3g} rms); {err:.3e} with the small floor; the oracle is {oracle_k:.3e} from f64")
    return exact_outputs
