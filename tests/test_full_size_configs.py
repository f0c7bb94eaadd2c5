"""The three model configurations at the size the benchmark times them, EVERY output element against the oracle, the
way the reference's `test_all` compares whole outputs (kn-cuda-eval/tests/root/runner.rs:10-55).

At these shapes the launch geometry is the timed one: 256-row matmul tiles over 512 tokens, four key blocks per query
tile of the fused attention, 16 M-tiles of the plane convolution over 1024 boards, the tail-split and grouped launches.
The reduced-size cases of `cases_graphs.py` exercise the same builders but none of these tilings.

The oracle is one thread per call. Positions of the ResNet batch and samples of the UNet batch do not depend on each
other, so their oracle runs are spread over a few threads (the same computation per position, the library call releases
the interpreter lock); the LLaMA prefill is one call.
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from kyanite_amd import HipExecutor, configs
from oracle import cpu_eval_graph
from runner import PARITY_RECORDS, check_outputs

pytestmark = pytest.mark.gpu

WORKERS = max(1, min(16, os.cpu_count() or 1))


def _oracle_in_chunks(graph_for, chunk_inputs):
    """`cpu_eval_graph` on independent parts of a batch side by side; returns the outputs joined along axis 0."""
    def run(part):
        graph, batch, inputs = graph_for(part), part[0], part[1]
        return cpu_eval_graph(graph, batch, inputs)
    with ThreadPoolExecutor(max_workers=WORKERS) as pool:
        results = list(pool.map(run, chunk_inputs))
    return [np.concatenate([r[i] for r in results], axis=0) for i in range(len(results[0]))]


def test_resnet_tower_batch_1024(hip_device):
    """configs[2]: all 1024 positions, policy [1024, 4672] and value [1024, 1]"""
    batch, chunk = 1024, 64
    graph, make_inputs, _ = configs.build_resnet_tower(seed=0)
    inputs = make_inputs(batch)
    print("resnet tower, batch 1024: gpu", flush=True)
    gpu = HipExecutor(hip_device, graph, batch).evaluate(inputs)
    print("resnet tower, batch 1024: oracle", flush=True)
    parts = [(chunk, [x[i:i + chunk] for x in inputs]) for i in range(0, batch, chunk)]
    expected = _oracle_in_chunks(lambda part: graph, parts)
    assert expected[0].shape == (batch, 4672) and expected[1].shape == (batch, 1)
    check_outputs(graph, batch, inputs, expected, gpu, "resnet tower, batch 1024, every position", PARITY_RECORDS)


def test_llama_decoder_512_tokens(hip_device):
    """configs[3]: all 512 tokens of the 2 layer decoder at d_model 4096"""
    graph, make_inputs, _ = configs.build_llama(seed=0)
    inputs = make_inputs()
    print("llama decoder, 512 tokens: gpu", flush=True)
    gpu = HipExecutor(hip_device, graph, 0).evaluate(inputs)
    print("llama decoder, 512 tokens: oracle (about a minute on one core)", flush=True)
    expected = cpu_eval_graph(graph, 0, inputs)
    assert expected[0].shape == (1, 512, 4096)
    check_outputs(graph, 0, inputs, expected, gpu, "llama decoder, 512 tokens, every token", PARITY_RECORDS)


def test_unet_block_batch_2(hip_device):
    """configs[4]: both samples at 64 x 64"""
    graph, make_inputs, _ = configs.build_unet_block(seed=0)
    inputs = make_inputs()
    print("unet block, batch 2: gpu", flush=True)
    gpu = HipExecutor(hip_device, graph, 0).evaluate(inputs)
    print("unet block, batch 2: oracle", flush=True)
    single = configs.build_unet_block(seed=0, batch=1)[0]
    parts = [(0, [x[i:i + 1] for x in inputs]) for i in range(2)]
    expected = _oracle_in_chunks(lambda part: single, parts)
    assert expected[0].shape == (2, 320, 64, 64)
    check_outputs(graph, 0, inputs, expected, gpu, "unet block, batch 2, both samples", PARITY_RECORDS)


# ---------------------------------------------------------------------------------------------------------------------
# Config 4 operation by operation. End to end the f16 decoder drifts: every stored value is rounded to 11 bits and the
# roundings of 14 stages pile up on both sides, so the whole-graph check above rests on the f64-referenced rule. Here
# each stage of layer 1 is a graph of its own at the full shape (512 tokens, d_model 4096, 32 heads, FFN 11008, the
# decoder's own weights), and BOTH sides get the ORACLE's value of the previous stage as input (teacher forcing): what
# is compared is one stage's kernels, with no drift from the stages before.

def _llama_stage_graphs(seed=0, seq=512, d_model=4096, heads=32, ffn=11008, eps=1e-6, rope_base=10000.0):
    """[(name, graph, names of its inputs, names of its outputs)] for layer 1 of `configs.build_llama`, with the same
    weight streams (401..407) and the same spelling of every operation."""
    import math

    from kyanite_amd import BinaryOp, DType, Graph, ReduceOp, UnaryOp
    from kyanite_amd.configs import cached_normal

    dt, np_dt = DType.F16, np.float16
    d_head = d_model // heads
    half = d_head // 2

    def weight(g, stream, co, ci):
        return g.constant([co, ci], cached_normal(seed, stream, (co, ci), 0.02, np_dt))

    def const(g, shape, array):
        return g.constant(list(shape), np.ascontiguousarray(array).astype(np_dt))

    def rmsnorm(g, x):
        ms = g.view(g.reduce(g.mul(x, x), [1], ReduceOp.MEAN), [seq, 1])
        rms = g.unary(UnaryOp.SQRT, g.add(ms, g.scalar(eps, dt)))
        return g.mul(g.binary(BinaryOp.DIV, x, rms), const(g, (1, d_model), np.ones((1, d_model))))

    inv_freq = rope_base ** (-np.arange(half, dtype=np.float64) * 2.0 / d_head)
    angles = np.arange(seq, dtype=np.float64)[:, None] * inv_freq[None, :]

    def rotary(g, t):
        cos_t, sin_t = const(g, (1, seq, half), np.cos(angles)[None]), const(g, (1, seq, half), np.sin(angles)[None])
        a, b = g.slice(t, 2, 0, half), g.slice(t, 2, half, d_head)
        return g.concat([g.sub(g.mul(a, cos_t), g.mul(b, sin_t)), g.add(g.mul(b, cos_t), g.mul(a, sin_t))], 2)

    def split_heads(g, t):
        return g.permute(g.view(t, [seq, heads, d_head]), [1, 0, 2])

    stages = []

    g = Graph()
    g.output(rmsnorm(g, g.input([seq, d_model], dt)))
    stages.append(("rmsnorm 1", g, ["x"], ["h"]))

    g = Graph()
    h = g.input([seq, d_model], dt)
    g.output(rotary(g, split_heads(g, g.linear(h, weight(g, 401, d_model, d_model)))))
    g.output(rotary(g, split_heads(g, g.linear(h, weight(g, 402, d_model, d_model)))))
    g.output(split_heads(g, g.linear(h, weight(g, 403, d_model, d_model))))
    stages.append(("q k v projections with rotary", g, ["h"], ["q", "k", "v"]))

    g = Graph()
    q, k, v = (g.input([heads, seq, d_head], dt) for _ in range(3))
    mask = const(g, (1, seq, seq), np.where(np.tril(np.ones((seq, seq), bool)), 0.0, -np.inf))
    scores = g.batched_mat_mul(q, g.permute(k, [0, 2, 1]))
    probs = g.softmax(g.add(g.mul(scores, g.scalar(1.0 / math.sqrt(d_head), dt)), mask), 2)
    g.output(g.view(g.permute(g.batched_mat_mul(probs, v), [1, 0, 2]), [seq, d_model]))
    stages.append(("causal attention", g, ["q", "k", "v"], ["ctx"]))

    g = Graph()
    ctx, x = g.input([seq, d_model], dt), g.input([seq, d_model], dt)
    g.output(g.add(x, g.linear(ctx, weight(g, 404, d_model, d_model))))
    stages.append(("o projection + residual", g, ["ctx", "x"], ["x1"]))

    g = Graph()
    g.output(rmsnorm(g, g.input([seq, d_model], dt)))
    stages.append(("rmsnorm 2", g, ["x1"], ["h2"]))

    g = Graph()
    h2 = g.input([seq, d_model], dt)
    gate, up = g.linear(h2, weight(g, 405, ffn, d_model)), g.linear(h2, weight(g, 406, ffn, d_model))
    g.output(g.mul(g.mul(gate, g.sigmoid(gate)), up))
    stages.append(("gate / up projections with SwiGLU", g, ["h2"], ["act"]))

    g = Graph()
    act, x1 = g.input([seq, ffn], dt), g.input([seq, d_model], dt)
    g.output(g.add(x1, g.linear(act, weight(g, 407, d_model, ffn))))
    stages.append(("down projection + residual", g, ["act", "x1"], ["x2"]))
    return stages


# What each stage is held to:
#   * the rules of oracle/parity.py like every other graph (`direct`, else the f64-referenced rule), with the
#     agreement rule (2) in force, not waived;
#   * `floor_needed`: how far below the tensor's rms an element must lie before GPU and oracle stop agreeing to 2e-2 of
#     it, against a bound derived per stage below;
#   * how many elements lie outside 2e-2 under the small floor (1e-3 rms) at all.
# Why a floor above 1e-3 rms is unavoidable in f16 even for a single matmul: both sides sum in f32 and round ONCE to f16,
# but in different orders, so an f32 sum that lies next to a rounding boundary lands on either neighbour: a few elements
# in a thousand differ by one f16 ulp, 2^-10 of a value y that may be several rms large. Where the stage then adds a
# residual (x + y) or rotates (a cos - b sin), the result can be far smaller than y, and one ulp of y is not small
# relative to it. The floor at which 2e-2 holds again is ulp16(max |y|) / 2e-2 over the output's rms: 2^-10 / 2e-2 =
# 0.049 for max |y| in [1, 2) and an rms of 1, which is what these stages measure (0.038 to 0.045).
# The fused attention is the one stage where the ORACLE's chain of separately rounded operations is the noisy side
# (scores up to 64 in magnitude are rounded to f16, ulp 2^-5, which after the scaling by 1 / sqrt(128) is 2.8e-3 in the
# exponent; early tokens, whose softmax has few terms, feel single flips): it is held to the f64 evaluation instead,
# where the GPU result may need no larger floor than the oracle's does.

def _ulp16(v):
    """the spacing of f16 values at magnitude v (normal range)"""
    return 2.0 ** (np.floor(np.log2(max(float(v), 2.0 ** -14))) - 10)


def _stage_floor_bound(name, inputs, e):
    """(bound on `floor_needed` in units of rms(e), largest fraction of elements outside 2e-2 under the small floor)"""
    e64 = e.astype(np.float64)
    rms = float(np.sqrt(np.mean(e64 * e64)))
    bar = 2e-2
    if name in ("o projection + residual", "down projection + residual"):
        y = e64 - inputs[1].astype(np.float64)  # the matmul result, to within the rounding of the sum
        return 1.05 * _ulp16(np.abs(y).max()) / bar / rms, 1e-4
    if name == "q k v projections with rotary":
        # a cos - b sin: a flip of a or b by one ulp, passed on through the rounded product: two ulps of the largest entry
        # (entries of the rotated pair are at most sqrt(2) times the largest output)
        return 2 * _ulp16(np.sqrt(2.0) * np.abs(e64).max()) / bar / rms, 1e-4
    return 1e-3, 0.0


def test_llama_layer_stage_by_stage(hip_device):
    from oracle.f64_eval import eval_graph_f64
    from oracle.parity import F16_MAX_REL, floor_needed

    stages = _llama_stage_graphs()
    values = {"x": configs.normal(0, 399, (1, 512, 4096))[0].astype(np.float16)}
    report, failures = [], []
    for name, graph, ins, outs in stages:
        inputs = [values[n] for n in ins]
        print(f"llama stage '{name}': gpu", flush=True)
        ex = HipExecutor(hip_device, graph, 0)
        gpu = ex.evaluate(inputs)
        print(f"llama stage '{name}': oracle; steps {ex.step_kinds()}", flush=True)
        expected = cpu_eval_graph(graph, 0, inputs)
        records = []
        exact = check_outputs(graph, 0, inputs, expected, gpu, f"llama layer 1, teacher forced: {name}", records)
        for out_name, e, a, record in zip(outs, expected, gpu, records):
            assert e.dtype == np.float16 and a.dtype == np.float16 and e.shape == a.shape
            e64, a64 = e.astype(np.float64).reshape(-1), a.astype(np.float64).reshape(-1)
            rms = float(np.sqrt(np.mean(e64 * e64)))
            over = int(np.count_nonzero(np.abs(a64 - e64) / np.maximum(np.abs(e64), 1e-3 * rms) > F16_MAX_REL))
            differ = int(np.count_nonzero(e64 != a64))
            needed = floor_needed(e, a, F16_MAX_REL)
            what = f"{record['what']} -> {out_name}"
            if name == "causal attention":
                if exact is None:
                    exact = eval_graph_f64(graph, 0, inputs)
                t = exact[record["output"]]
                needed_gpu, needed_oracle = floor_needed(t, a, F16_MAX_REL), floor_needed(t, e, F16_MAX_REL)
                record.update(floor_needed_gpu_vs_f64=needed_gpu, floor_needed_oracle_vs_f64=needed_oracle)
                print(f"    {out_name}: against f64 the GPU needs a floor of {needed_gpu:.4f} rms, the oracle {needed_oracle:.4f}", flush=True)
                if needed_gpu > 1.25 * needed_oracle:
                    failures.append(f"{what}: against f64 the GPU needs a floor of {needed_gpu:.4f} rms, the oracle only {needed_oracle:.4f}")
                bound, over_bound = 0.5, 2e-2
            else:
                bound, over_bound = _stage_floor_bound(name, inputs, e)
                if record.get("rule2_waived"):
                    failures.append(f"{what}: the agreement rule was waived")
            record.update(what=what, floor_bound=bound, elements_over_bar_small_floor=over, elements_that_differ=differ)
            print(f"    {out_name}: rule {record['rule']}, max rel err {record['err']:.3e} under the 1e-3 rms floor, floor needed "
                  f"{needed:.4f} rms (bound {bound:.4f}), {over} of {e.size} outside 2e-2 under the small floor, "
                  f"{differ} differ at all, rule 2 waived: {record.get('rule2_waived', False)}", flush=True)
            if needed > bound:
                failures.append(f"{what}: needs a floor of {needed:.4f} rms, bound {bound:.4f}")
            if over > over_bound * e.size:
                failures.append(f"{what}: {over} of {e.size} elements outside 2e-2 under the small floor, bound {over_bound:.0e} of them")
            values[out_name] = e  # the ORACLE's value feeds the next stage on both sides
        report.extend(records)
        del ex
    PARITY_RECORDS.extend(report)
    assert not failures, "\n".join(failures)
