"""Graph blobs that cross the C ABI (knhip_graph_deserialize, knhip_executor_new_from_blob) are checked value by
value: a blob whose stored shapes, dtypes or axes are not what its operations yield is refused before any host-side
query or the planner sees it. The rules are those of the builder methods (graph.rs:617-1269 on the reference side).
Runs without a GPU."""
import struct

import numpy as np
import pytest

from kyanite_amd import Graph, KnError

F32, I32, F16 = 0, 4, 11
INPUT, CONSTANT, VIEW, BROADCAST, PERMUTE, SLICE, FLIP, GATHER, CONCAT, CONV, MATMUL, UNARY, BINARY, SOFTMAX, LAYERNORM, REDUCE = range(16)


def u32(*v):
    return struct.pack("<%dI" % len(v), *v)


def u64(*v):
    return struct.pack("<%dQ" % len(v), *v)


def value(dtype, shape, kind, payload):
    out = bytes([dtype]) + u32(len(shape))
    for d in shape:
        factor, exp = d if isinstance(d, tuple) else (d, 0)
        out += u64(factor) + u32(exp)
    return out + bytes([kind]) + payload + u32(0)


def blob(values, inputs, outputs):
    return u32(0x47484E4B, 1, len(values)) + b"".join(values) + u32(len(inputs), *inputs) + u32(len(outputs), *outputs)


def inp(shape, index=0, dtype=F32):
    return value(dtype, shape, INPUT, u32(index))


def load(values, n_inputs=1):
    return Graph.from_bytes(blob(values, list(range(n_inputs)), [len(values) - 1]))


GOOD = {
    "view": [inp([4, 6]), value(F32, [3, 8], VIEW, u32(0))],
    "broadcast": [inp([1, 6]), value(F32, [5, 6], BROADCAST, u32(0))],
    "permute": [inp([2, 3, 4]), value(F32, [4, 2, 3], PERMUTE, u32(0, 3, 2, 0, 1))],
    "slice": [inp([4, 10]), value(F32, [4, 3], SLICE, u32(0, 1) + u64(1, 10, 3))],
    "flip": [inp([4, 6]), value(F32, [4, 6], FLIP, u32(0, 1))],
    "softmax": [inp([4, 6]), value(F32, [4, 6], SOFTMAX, u32(0, 1))],
    "layernorm": [inp([4, 6]), value(F32, [4, 6], LAYERNORM, u32(0, 1) + struct.pack("<f", 1e-5))],
    "gather": [inp([4, 6]), inp([3], 1, I32), value(F32, [4, 3], GATHER, u32(0, 1, 1))],
    "concat": [inp([4, 6]), inp([4, 2], 1), value(F32, [4, 8], CONCAT, u32(2, 0, 1, 1))],
    "matmul": [inp([2, 3, 4]), inp([2, 4, 5], 1), value(F32, [2, 3, 5], MATMUL, u32(0, 1))],
    "unary": [inp([4, 6]), value(F32, [4, 6], UNARY, u32(0) + bytes([4, 0]))],
    "binary": [inp([4, 6]), inp([4, 6], 1), value(F32, [4, 6], BINARY, u32(0, 1) + bytes([0]))],
    "reduce": [inp([4, 6, 5]), value(F32, [6], REDUCE, u32(0, 2, 0, 2) + bytes([0]))],
    "conv": [inp([(1, 1), 3, 8, 8]), inp([5, 3, 3, 3], 1),
             value(F32, [(1, 1), 5, 8, 8], CONV, u32(0, 1) + u64(1, 1, 1, 1, 3, 3, 8, 8))],
}
N_INPUTS = {"gather": 2, "concat": 2, "matmul": 2, "binary": 2, "conv": 2}


@pytest.mark.parametrize("name", sorted(GOOD))
def test_well_formed_blobs_load(name):
    g = load(GOOD[name], N_INPUTS.get(name, 1))
    assert Graph.from_bytes(g.to_bytes()).to_bytes() == g.to_bytes()


BAD = {
    "view size": [inp([4, 6]), value(F32, [3, 7], VIEW, u32(0))],
    "view dtype": [inp([4, 6]), value(I32, [4, 6], VIEW, u32(0))],
    "broadcast rank": [inp([6]), value(F32, [5, 6], BROADCAST, u32(0))],
    "broadcast axis": [inp([2, 6]), value(F32, [5, 6], BROADCAST, u32(0))],
    "permute repeats": [inp([2, 3, 4]), value(F32, [4, 2, 2], PERMUTE, u32(0, 3, 2, 0, 0))],
    "permute out of range": [inp([2, 3, 4]), value(F32, [4, 2, 3], PERMUTE, u32(0, 3, 2, 0, 3))],
    "permute shape": [inp([2, 3, 4]), value(F32, [2, 3, 4], PERMUTE, u32(0, 3, 2, 0, 1))],
    "slice past the end": [inp([4, 10]), value(F32, [4, 4], SLICE, u32(0, 1) + u64(1, 13, 3))],
    "slice axis": [inp([4, 10]), value(F32, [4, 3], SLICE, u32(0, 2) + u64(1, 10, 3))],
    "slice shape": [inp([4, 10]), value(F32, [4, 4], SLICE, u32(0, 1) + u64(1, 10, 3))],
    "flip axis": [inp([4, 6]), value(F32, [4, 6], FLIP, u32(0, 2))],
    "softmax axis": [inp([4, 6]), value(F32, [4, 6], SOFTMAX, u32(0, 7))],
    "softmax shape": [inp([4, 6]), value(F32, [4, 7], SOFTMAX, u32(0, 1))],
    "softmax of integers": [inp([4, 6], 0, I32), value(I32, [4, 6], SOFTMAX, u32(0, 1))],
    "layernorm axis": [inp([4, 6]), value(F32, [4, 6], LAYERNORM, u32(0, 2) + struct.pack("<f", 1e-5))],
    "gather float indices": [inp([4, 6]), inp([3], 1, F32), value(F32, [4, 3], GATHER, u32(0, 1, 1))],
    "gather indices rank": [inp([4, 6]), inp([3, 1], 1, I32), value(F32, [4, 3], GATHER, u32(0, 1, 1))],
    "gather shape": [inp([4, 6]), inp([3], 1, I32), value(F32, [4, 6], GATHER, u32(0, 1, 1))],
    "concat sum": [inp([4, 6]), inp([4, 2], 1), value(F32, [4, 9], CONCAT, u32(2, 0, 1, 1))],
    "concat off axis": [inp([4, 6]), inp([3, 2], 1), value(F32, [4, 8], CONCAT, u32(2, 0, 1, 1))],
    "concat axis": [inp([4, 6]), inp([4, 2], 1), value(F32, [4, 8], CONCAT, u32(2, 0, 1, 2))],
    "matmul inner": [inp([2, 3, 4]), inp([2, 5, 5], 1), value(F32, [2, 3, 5], MATMUL, u32(0, 1))],
    "matmul n": [inp([2, 3, 4]), inp([2, 4, 5], 1), value(F32, [2, 3, 6], MATMUL, u32(0, 1))],
    "matmul rank": [inp([3, 4]), inp([4, 5], 1), value(F32, [3, 5], MATMUL, u32(0, 1))],
    "matmul dtype": [inp([2, 3, 4]), inp([2, 4, 5], 1, F16), value(F32, [2, 3, 5], MATMUL, u32(0, 1))],
    "unary dtype": [inp([4, 6]), value(I32, [4, 6], UNARY, u32(0) + bytes([4, 0]))],
    "unary exp of integers": [inp([4, 6], 0, I32), value(I32, [4, 6], UNARY, u32(0) + bytes([4, 0]))],
    "unary shape": [inp([4, 6]), value(F32, [6, 4], UNARY, u32(0) + bytes([4, 0]))],
    "binary not broadcast": [inp([4, 6]), inp([1, 6], 1), value(F32, [4, 6], BINARY, u32(0, 1) + bytes([0]))],
    "binary dtype": [inp([4, 6]), inp([4, 6], 1, I32), value(F32, [4, 6], BINARY, u32(0, 1) + bytes([0]))],
    "reduce axis": [inp([4, 6, 5]), value(F32, [6], REDUCE, u32(0, 2, 0, 3) + bytes([0]))],
    "reduce repeats": [inp([4, 6, 5]), value(F32, [6, 5], REDUCE, u32(0, 2, 0, 0) + bytes([0]))],
    "reduce shape": [inp([4, 6, 5]), value(F32, [4], REDUCE, u32(0, 2, 0, 2) + bytes([0]))],
    "conv output shape": [inp([(1, 1), 3, 8, 8]), inp([5, 3, 3, 3], 1),
                          value(F32, [(1, 1), 4, 8, 8], CONV, u32(0, 1) + u64(1, 1, 1, 1, 3, 3, 8, 8))],
    "conv output size": [inp([(1, 1), 3, 8, 8]), inp([5, 3, 3, 3], 1),
                         value(F32, [(1, 1), 5, 9, 8], CONV, u32(0, 1) + u64(1, 1, 1, 1, 3, 3, 9, 8))],
    "conv even kernel": [inp([(1, 1), 3, 8, 8]), inp([5, 3, 2, 2], 1),
                         value(F32, [(1, 1), 5, 7, 7], CONV, u32(0, 1) + u64(1, 1, 0, 0, 2, 2, 7, 7))],
    "operand is not earlier": [inp([4, 6]), value(F32, [4, 6], FLIP, u32(1, 1))],
}
BAD_INPUTS = {"gather float indices": 2, "gather indices rank": 2, "gather shape": 2, "concat sum": 2, "concat off axis": 2,
              "concat axis": 2, "matmul inner": 2, "matmul n": 2, "matmul rank": 2, "matmul dtype": 2,
              "binary not broadcast": 2, "binary dtype": 2, "conv output shape": 2, "conv output size": 2, "conv even kernel": 2}


@pytest.mark.parametrize("name", sorted(BAD))
def test_inconsistent_blobs_are_refused(name):
    with pytest.raises(KnError):
        load(BAD[name], BAD_INPUTS.get(name, 1))


def test_bytes_flipped_in_real_graphs_never_load_as_something_else():
    """Every single-byte change of the structural part of a real blob either fails to load or loads as a graph that
    serialises to exactly the changed bytes (a different, but consistent, graph): nothing is silently repaired."""
    from cases_graphs import CASES
    rng = np.random.default_rng(5)
    for name in ("attention_block", "layernorm_fused", "gather_real"):
        data = CASES[name]()[0].to_bytes()
        refused = 0
        for pos in rng.choice(len(data), size=300, replace=False):
            changed = bytearray(data)
            changed[pos] ^= 1 << int(rng.integers(0, 8))
            try:
                g = Graph.from_bytes(bytes(changed))
            except KnError:
                refused += 1
                continue
            assert g.to_bytes() == bytes(changed), (name, int(pos))
        assert refused > 0
