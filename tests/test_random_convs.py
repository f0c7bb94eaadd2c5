"""Differential test on seeded random convolutions: image sizes (powers of two, board sizes, odd rectangles), channel
counts (multiples of 8 and not, fewer than a tile and more), batches from one image to a few tiles, filters of 1 x 1,
3 x 3, 5 x 5, 1 x 3 and 3 x 1, strides of 1 and 2, padding of none and "same", and bias / residual / activation in the
store. Together they reach every launch the convolution takes: planes of power-of-two images, planes of any image
size (float by float and four floats at a time), the patch kernel, 1 x 1 as a matrix product, both tile sizes, and the
input channels in slices when the tiles are few.

CPU half: the graph evaluates in the oracle and plans for gfx950. GPU half: `check_gpu` against the oracle.
"""
import numpy as np
import pytest

from kyanite_amd import Graph
from runner import check_cpu, check_gpu

SEEDS = list(range(64))


def build(seed):
    rng = np.random.default_rng(9000 + seed)
    pick = lambda options: options[int(rng.integers(len(options)))]
    g = Graph()
    inputs = []

    def tensor(shape, scale, constant=False):
        data = (rng.standard_normal(shape) * scale).astype(np.float32)
        if constant:
            return g.constant(list(shape), data)
        inputs.append(data)
        return g.input(list(shape))

    h, w = pick([(8, 8), (16, 16), (4, 32), (9, 9), (7, 7), (19, 19), (5, 3), (12, 20), (28, 28), (11, 6), (3, 3), (33, 31)])
    kh, kw = pick([(3, 3), (3, 3), (3, 3), (1, 1), (5, 5), (1, 3), (3, 1)])
    stride = pick([1, 1, 1, 2])
    same = pick([True, True, False])
    pad_y, pad_x = (kh // 2, kw // 2) if same else (0, 0)
    if h + 2 * pad_y < kh or w + 2 * pad_x < kw:
        pad_y, pad_x = kh // 2, kw // 2
    in_c = pick([1, 3, 8, 16, 21, 40, 64, 72, 136])
    out_c = pick([1, 5, 8, 32, 64, 70, 128, 130])
    oh, ow = (h + 2 * pad_y - kh) // stride + 1, (w + 2 * pad_x - kw) // stride + 1
    batch = pick([1, 2, 5, 16, 37])
    # keep the oracle's share of the test run in seconds
    while batch > 1 and batch * oh * ow * out_c * in_c * kh * kw > 6e7:
        batch = max(1, batch // 2)
    x = tensor((batch, in_c, h, w), 1.0)
    y = g.conv(x, tensor((out_c, in_c, kh, kw), 1.0 / np.sqrt(in_c * kh * kw), constant=True), stride, stride, pad_y, pad_x)
    epilogue = pick(["none", "bias", "bias_relu", "bias_residual_relu", "relu"])
    if "bias" in epilogue:
        y = g.add(y, tensor((1, out_c, 1, 1), 1.0, constant=True))
    if "residual" in epilogue:
        y = g.add(y, tensor((batch, out_c, oh, ow), 1.0))
    if "relu" in epilogue:
        y = g.relu(y)
    g.output(y)
    return g, inputs


@pytest.mark.parametrize("seed", SEEDS)
def test_cpu(seed):
    g, inputs = build(seed)
    check_cpu(g, 0, inputs, None)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", SEEDS)
def test_gpu(seed, hip_device):
    g, inputs = build(seed)
    check_gpu(hip_device, g, 0, inputs, None, what=f"random conv {seed}")
