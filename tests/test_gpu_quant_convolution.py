"""GPU parity of quant_convolution (the direct kernel, or im2col + the quantized GEMM; one to three spatial axes) through
the C ABI against the CPU oracle: int32 results bit-exact, dequantized results bit-exact for int8, fp8 within the
accumulation tolerance of the fp8 matrix instructions."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev, half_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def test_reference_known_answers_on_gpu(ops, golden):
    for c in golden["convolution"]:
        if c["type"] != "int8":
            continue
        x = np.arange(int(np.prod(c["x_lens"]))).astype(np.int8).reshape(c["x_lens"])
        w = np.arange(int(np.prod(c["w_lens"]))).astype(np.int8).reshape(c["w_lens"])
        got = ops.quant_convolution(dev(x), dev(w), c["padding"], c["stride"], c["dilation"], c["group"])
        assert got.dtype == torch.int32
        assert got.cpu().numpy().flatten().tolist() == c["gold"], c["name"]


CASES = [
    # x shape, w shape, padding, stride, dilation, group
    ((2, 64, 14, 14), (64, 64, 3, 3), (1, 1), (1, 1), (1, 1), 1),      # K = 576: no padding of K
    ((1, 3, 33, 31), (16, 3, 7, 7), (3, 3), (2, 2), (1, 1), 1),        # K = 147 -> 192
    ((3, 32, 9, 12), (48, 32, 1, 1), (0, 0), (1, 1), (1, 1), 1),       # pointwise
    ((2, 16, 10, 10), (24, 4, 3, 3), (2, 1), (1, 2), (2, 1), 4),       # groups, dilation, mixed pads
    ((1, 8, 12, 12), (8, 1, 3, 3), (1, 1), (1, 1), (1, 1), 8),         # depthwise
    ((2, 5, 1, 40), (7, 5, 1, 5), (0, 2), (1, 3), (1, 1), 1),          # one-dimensional
    ((1, 20, 6, 6), (300, 20, 3, 3), (0, 0), (1, 1), (1, 1), 1),       # more than one row tile of weights
    ((2, 8, 9, 10), (8, 8, 3, 3), (0, 1, 2, 0), (2, 2), (1, 1), 1),    # low and high padding differ
    # 16 | channels per group, two groups
    ((2, 64, 9, 11), (32, 32, 3, 2), (1, 0, 2, 1), (2, 1), (1, 2), 2),
    ((1, 16, 7, 7), (5, 16, 5, 5), (2, 2), (1, 1), (1, 1), 1),         # K = 400 -> 448
    ((3, 48, 6, 5), (7, 48, 2, 2), (0, 0), (1, 1), (1, 1), 1),
    # one image, deep K, one output tile: the GEMM splits K inside the convolution's workspace
    ((1, 256, 14, 14), (256, 256, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((1, 128, 12, 12), (96, 64, 5, 5), (2, 2), (1, 1), (1, 1), 2),
    ((1, 512, 7, 7), (64, 512, 3, 3), (1, 1), (1, 1), (1, 1), 1),      # 49 positions: N % 4 != 0 in the split
    # the direct kernel (int8, 16 | channels per group): channel tiles with a ragged end, row tiles that
    # straddle images, K steps with a zero-filled second half, windows over the zero border only
    ((3, 32, 10, 13), (80, 32, 3, 3), (1, 1), (1, 1), (1, 1), 1),      # 80 channels: tiles of 64 + 16; 130 positions
    ((2, 96, 8, 8), (144, 48, 3, 3), (2, 2), (1, 1), (2, 2), 2),       # 72 channels per group, dilation, K = 432 -> 512
    ((5, 16, 6, 6), (16, 16, 2, 2), (3, 3), (2, 2), (1, 1), 1),        # padding wider than the window
    ((4, 64, 56, 56), (64, 64, 3, 3), (1, 1), (1, 1), (1, 1), 1),      # the benchmark's first layer shape, 4 images
    ((4, 256, 14, 14), (256, 256, 3, 3), (1, 1), (1, 1), (1, 1), 1),   # and its second
    ((2, 128, 28, 28), (128, 128, 3, 3), (1, 1), (2, 2), (1, 1), 1),   # stride 2
    # windows of one element, unit strides, no padding: the GEMM on the tensors as they lie (row-major second operand)
    ((2, 64, 28, 28), (128, 64, 1, 1), (0, 0), (1, 1), (1, 1), 1),     # 784 positions: the direct-to-LDS GEMM
    ((3, 128, 16, 16), (96, 64, 1, 1), (0, 0), (1, 1), (1, 1), 2),     # two groups
    ((2, 40, 7, 9), (24, 40, 1, 1), (0, 0), (1, 1), (3, 2), 1),        # 63 positions, 40 channels: the general GEMM
    ((2, 64, 14, 14), (96, 64, 1, 1), (0, 0), (2, 2), (1, 1), 1),      # 1 x 1 with strides: the direct kernel subsamples
    # not the direct kernel's form (two groups of 100 channels): one image of a deep layer through im2col and the
    # GEMM's split K
    ((1, 200, 7, 7), (64, 100, 3, 3), (1, 1), (1, 1), (1, 1), 2),
    # many groups of few channels (one thread per output): depthwise with strides, groups of 3 with dilation
    ((3, 48, 15, 17), (48, 1, 3, 3), (1, 1), (2, 2), (1, 1), 48),
    ((2, 24, 9, 9), (40, 3, 3, 3), (2, 2), (1, 1), (2, 2), 8),
    # the same kernel's four-outputs-of-a-row form (unit stride and dilation along x, at most 4 columns): a window
    # 4 wide with padding 2 and a ragged last group, one column, and 5 columns (one output per thread again)
    ((2, 12, 9, 10), (12, 1, 3, 4), (1, 2), (1, 1), (1, 1), 12),
    ((1, 6, 5, 3), (6, 1, 3, 1), (1, 0), (2, 1), (1, 1), 6),
    ((2, 12, 9, 11), (24, 2, 2, 5), (0, 2), (1, 1), (1, 1), 6),
    # depthwise over images with unit stride along x: rows staged in LDS.  Dword-aligned rows; several row chunks per
    # plane with a strided, dilated 5 x 4 window and 4 columns of padding; two output channels per input channel;
    # no padding on the left
    ((2, 16, 28, 28), (16, 1, 3, 3), (1, 1), (1, 1), (1, 1), 16),
    ((1, 2, 300, 64), (2, 1, 5, 4), (3, 4), (2, 1), (2, 1), 2),
    ((2, 8, 12, 12), (16, 1, 3, 3), (1, 1), (1, 1), (1, 1), 8),
    ((1, 4, 20, 24), (4, 1, 3, 3), (0, 0, 2, 3), (1, 1), (1, 1), 4),
    # one group with any channel count: the direct kernel on a copy whose channels are rounded up to 16 (zeros)
    ((2, 3, 40, 36), (24, 3, 7, 7), (3, 3), (2, 2), (1, 1), 1),        # an image network's first layer
    # at most 4 channels in one group: pixels of 4 channels, K pieces of 4 window columns.  4 channels with a window
    # of exactly 4 columns and a dilated, strided y; one channel with 5 columns (the second piece reaches past the
    # window, and past the copy's end at the last row); 2 columns
    ((2, 4, 17, 19), (10, 4, 3, 4), (2, 1), (2, 1), (2, 1), 1),
    ((3, 1, 9, 12), (70, 1, 3, 5), (0, 0), (1, 1), (1, 1), 1),
    ((2, 2, 11, 8), (16, 2, 2, 2), (1, 0, 0, 1), (1, 2), (1, 1), 1),
    ((2, 24, 14, 14), (40, 24, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((1, 200, 7, 7), (64, 200, 3, 3), (1, 1), (1, 1), (1, 1), 1),      # 200 -> 208 channels
]


@pytest.mark.parametrize("xs,ws,padding,stride,dilation,group", CASES)
def test_int8_bit_exact(ops, xs, ws, padding, stride, dilation, group):
    rng = np.random.default_rng(sum(xs) * 7 + sum(ws))
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    want = orc.convolution(x, w, orc.I8, padding, stride, dilation, group)
    print("conv int8", xs, ws, padding, stride, dilation, group, flush=True)
    got = ops.quant_convolution(dev(x), dev(w), padding, stride, dilation, group)
    assert tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("per_channel", [False, True])
def test_int8_dequant_epilogue_bit_exact(ops, out, per_channel):
    """quant_convolution -> dequantizelinear(scale_x * scale_w[o]) [-> convert], the graph
    simplify_qdq.cpp:171-222 leaves for symmetric zero points."""
    rng = np.random.default_rng(5)
    xs, ws = (2, 32, 12, 12), (40, 16, 3, 3)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    sx = np.float32(0.0213)
    sw = rng.uniform(0.001, 0.01, 40 if per_channel else 1).astype(np.float32)
    acc = orc.convolution(x, w, orc.I8, (1, 1), (1, 1), (1, 1), 2)
    scale = (sx * sw).astype(np.float32)                      # the graph's fp32 `mul`
    scale_full = np.broadcast_to(scale.reshape(1, -1, 1, 1) if per_channel else scale.reshape(1, 1, 1, 1),
                                 acc.shape)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale_full), None, orc.I32, orc.F32)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    got = ops.quant_convolution(dev(x), dev(w), (1, 1), (1, 1), (1, 1), 2, scale_x=dev(np.float32([sx])),
                                scale_w=dev(sw), out_dtype=td)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        ot = orc.F16 if out == "f16" else orc.BF16
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, ot))


@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_direct_kernel_dequant_without_vector_stores(ops, out):
    """49 positions per image: a lane's four results are not one aligned vector of the NCHW result, so the direct
    kernel stores them one by one; two groups of 24 channels (a ragged channel tile), three images in one row tile."""
    rng = np.random.default_rng(16)
    xs, ws = (3, 64, 7, 7), (48, 32, 3, 3)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    sx = np.float32(0.0371)
    sw = rng.uniform(0.001, 0.01, 48).astype(np.float32)
    acc = orc.convolution(x, w, orc.I8, (1, 1), (1, 1), (1, 1), 2)
    scale = np.broadcast_to((sx * sw).astype(np.float32).reshape(1, -1, 1, 1), acc.shape)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.I32, orc.F32)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    got = ops.quant_convolution(dev(x), dev(w), (1, 1), (1, 1), (1, 1), 2, scale_x=dev(np.float32([sx])),
                                scale_w=dev(sw), out_dtype=td)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, orc.F16 if out == "f16" else orc.BF16))
    bare = ops.quant_convolution(dev(x), dev(w), (1, 1), (1, 1), (1, 1), 2)
    assert np.array_equal(bare.cpu().numpy(), acc)


@pytest.mark.parametrize("seed", range(24))
def test_seeded_random_layers_bit_exact(ops, seed):
    """Random layers over every form the entry point chooses between (one to three spatial axes, any channel counts,
    groups, windows, strides, dilations, low / high padding, batches that make row tiles straddle images): int32 sums
    equal to the oracle's."""
    rng = np.random.default_rng(1000 + seed)
    nd = int(rng.integers(1, 4))
    group = int(rng.choice([1, 1, 1, 2, 3, 8]))
    cg = int(rng.choice([1, 3, 5, 16, 24, 32, 48])) if group == 1 or rng.random() < 0.5 else int(rng.choice([1, 2, 16, 32]))
    og = int(rng.choice([1, 7, 16, 40, 70]))
    win = [int(rng.integers(1, 4)) for _ in range(nd)]
    stride = [int(rng.integers(1, 3)) for _ in range(nd)]
    dil = [int(rng.integers(1, 3)) for _ in range(nd)]
    pad_lo = [int(rng.integers(0, 3)) for _ in range(nd)]
    pad_hi = [int(rng.integers(0, 3)) for _ in range(nd)]
    size = [int(rng.integers(d * (k - 1) + 1, d * (k - 1) + 9)) for k, d in zip(win, dil)]
    n = int(rng.integers(1, 5))
    xs = (n, group * cg, *size)
    ws = (group * og, cg, *win)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    padding = tuple(pad_lo) + tuple(pad_hi)
    want = orc.convolution(x, w, orc.I8, padding, tuple(stride), tuple(dil), group)
    print("conv seeded", seed, xs, ws, padding, stride, dil, group, flush=True)
    got = ops.quant_convolution(dev(x), dev(w), padding, tuple(stride), tuple(dil), group)
    assert tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("size", [(11, 13), (12, 16)])
@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_depthwise_convolution_dequant_epilogue_and_fp8(ops, out, size):
    """One channel per group: the kernel that stages rows in LDS (bytewise, and in dwords for rows of 16) with the
    per-channel scale; fp8 operands on it give exact sums for small integers."""
    rng = np.random.default_rng(27)
    xs, ws = (2, 40, *size), (40, 1, 3, 3)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    sx = np.float32(0.0191)
    sw = rng.uniform(0.001, 0.01, 40).astype(np.float32)
    acc = orc.convolution(x, w, orc.I8, (1, 1), (1, 1), (1, 1), 40)
    scale = np.broadcast_to((sx * sw).astype(np.float32).reshape(1, -1, 1, 1), acc.shape)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.I32, orc.F32)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    got = ops.quant_convolution(dev(x), dev(w), (1, 1), (1, 1), (1, 1), 40, scale_x=dev(np.float32([sx])),
                                scale_w=dev(sw), out_dtype=td)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, orc.F16 if out == "f16" else orc.BF16))
    xi = rng.integers(-3, 4, xs).astype(np.float32)
    wi = rng.integers(-2, 3, ws).astype(np.float32)
    gotf = ops.quant_convolution(dev(orc.fp8_from_f32(xi)), dev(orc.fp8_from_f32(wi)), (1, 1), (1, 1), (1, 1), 40, fp8=True)
    assert np.array_equal(gotf.cpu().numpy(), orc.convolution(xi, wi, orc.F32, (1, 1), (1, 1), (1, 1), 40))
    # a NaN weight spoils the outputs whose window has that element inside the image only: products with the zero
    # border are left out, as in the reference's loop (op/convolution.hpp skips positions outside the input)
    wc = orc.fp8_from_f32(wi)
    wc[0, 0, 0, 0] = 0x7F
    wn = wi.copy()
    wn[0, 0, 0, 0] = np.nan
    gotn = ops.quant_convolution(dev(orc.fp8_from_f32(xi)), dev(wc), (1, 1), (1, 1), (1, 1), 40, fp8=True).cpu().numpy()
    wantn = orc.convolution(xi, wn, orc.F32, (1, 1), (1, 1), (1, 1), 40)
    assert np.isnan(wantn[:, 0, 1:, 1:]).all() and not np.isnan(wantn[:, 0, 0, :]).any()
    assert np.array_equal(gotn, wantn, equal_nan=True)
    xf = rng.standard_normal(xs).astype(np.float32)
    wf = (rng.standard_normal(ws) * 0.05).astype(np.float32)
    xq = orc.quantizelinear(xf.reshape(-1, xs[-1]), np.float32(np.abs(xf).max() / 448), None, orc.F32, orc.FP8).reshape(xs)
    wq = orc.quantizelinear(wf.reshape(-1, ws[-1]), np.float32(np.abs(wf).max() / 448), None, orc.F32, orc.FP8).reshape(ws)
    wantq = orc.convolution(xq, wq, orc.FP8, (1, 1), (1, 1), (1, 1), 40)
    mag = orc.convolution(np.abs(orc.fp8_to_f32(xq)).astype(np.float32), np.abs(orc.fp8_to_f32(wq)).astype(np.float32),
                          orc.F32, (1, 1), (1, 1), (1, 1), 40)
    gotq = ops.quant_convolution(dev(xq), dev(wq), (1, 1), (1, 1), (1, 1), 40, fp8=True).cpu().numpy()
    assert np.all(np.abs(gotq - wantq) <= np.maximum(1e-3 * np.abs(wantq), 2.0 ** -14 * mag))


@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_pointwise_convolution_dequant_epilogue(ops, out):
    """A 1 x 1 convolution is the quantized GEMM on the tensors as they lie; the per-output-channel scale is the
    GEMM's per-row scale.  Two groups, 256 positions."""
    rng = np.random.default_rng(26)
    xs, ws = (2, 128, 16, 16), (80, 64, 1, 1)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    sx = np.float32(0.0151)
    sw = rng.uniform(0.001, 0.01, 80).astype(np.float32)
    acc = orc.convolution(x, w, orc.I8, (0, 0), (1, 1), (1, 1), 2)
    scale = np.broadcast_to((sx * sw).astype(np.float32).reshape(1, -1, 1, 1), acc.shape)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.I32, orc.F32)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    got = ops.quant_convolution(dev(x), dev(w), (0, 0), (1, 1), (1, 1), 2, scale_x=dev(np.float32([sx])),
                                scale_w=dev(sw), out_dtype=td)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, orc.F16 if out == "f16" else orc.BF16))


@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_int8_dequant_epilogue_with_split_k(ops, out):
    """One image of a deep layer: K is split over the chip and the second kernel applies the
    per-output-channel scale (a row scale of the GEMM); same bits as the oracle."""
    rng = np.random.default_rng(6)
    xs, ws = (1, 256, 14, 14), (256, 256, 3, 3)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    sx = np.float32(0.0213)
    sw = rng.uniform(0.001, 0.01, 256).astype(np.float32)
    acc = orc.convolution(x, w, orc.I8, (1, 1), (1, 1), (1, 1), 1)
    scale = np.broadcast_to((sx * sw).astype(np.float32).reshape(1, -1, 1, 1), acc.shape)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.I32, orc.F32)
    td = torch.float32 if out == "f32" else torch.bfloat16
    got = ops.quant_convolution(dev(x), dev(w), (1, 1), (1, 1), (1, 1), 1, scale_x=dev(np.float32([sx])),
                                scale_w=dev(sw), out_dtype=td)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, orc.BF16))


VOLUME_CASES = [
    # x shape, w shape, padding, stride, dilation, group: three spatial axes, then one
    ((2, 4, 5, 6, 7), (6, 4, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),           # K = 108 -> 128
    ((1, 6, 6, 5, 4), (4, 3, 2, 3, 1), (1, 0, 2), (2, 1, 1), (1, 2, 1), 2),           # groups, strides, dilation
    ((2, 4, 7, 4, 5), (4, 1, 3, 2, 2), (0, 1, 0, 2, 0, 1), (1, 2, 3), (2, 1, 1), 4),  # depthwise, low / high padding
    ((1, 3, 4, 4, 4), (2, 3, 1, 1, 1), (0, 0, 0), (2, 2, 2), (1, 1, 1), 1),           # pointwise with strides
    ((2, 32, 4, 6, 5), (24, 16, 3, 3, 3), (1, 1, 1), (1, 2, 1), (1, 1, 1), 2),        # channels-last gather
    ((1, 16, 8, 7, 6), (40, 16, 2, 3, 2), (0, 1, 1, 1, 0, 0), (1, 1, 1), (2, 1, 2), 1),
    ((1, 64, 6, 6, 6), (64, 64, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),        # K = 1728: split K
    ((3, 2, 9), (4, 2, 3), (1,), (2,), (2,), 1),                                      # [N, C, W]
    ((2, 32, 40), (6, 16, 5), (2, 0), (1,), (3,), 2),
]


@pytest.mark.parametrize("xs,ws,padding,stride,dilation,group", VOLUME_CASES)
def test_int8_one_and_three_spatial_axes_bit_exact(ops, xs, ws, padding, stride, dilation, group):
    rng = np.random.default_rng(sum(xs) * 5 + sum(ws))
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    want = orc.convolution(x, w, orc.I8, padding, stride, dilation, group)
    print("conv int8", xs, ws, padding, stride, dilation, group, flush=True)
    got = ops.quant_convolution(dev(x), dev(w), padding, stride, dilation, group)
    assert got.dtype == torch.int32 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


def test_volume_of_depth_one_equals_the_image(ops):
    """The two-dimensional entry point and the three-dimensional one agree where they overlap."""
    rng = np.random.default_rng(12)
    x = rng.integers(-128, 128, (2, 16, 9, 8), dtype=np.int8)
    w = rng.integers(-128, 128, (12, 16, 3, 3), dtype=np.int8)
    flat = ops.quant_convolution(dev(x), dev(w), (1, 0), (1, 2), (1, 1))
    vol = ops.quant_convolution(dev(x[:, :, None]), dev(w[:, :, None]), (0, 1, 0), (1, 1, 2), (1, 1, 1))
    assert torch.equal(vol[:, :, 0], flat)


def test_three_axis_dequant_epilogue_and_fp8(ops):
    rng = np.random.default_rng(13)
    xs, ws = (2, 16, 5, 6, 6), (20, 16, 3, 3, 3)
    x = rng.integers(-128, 128, xs, dtype=np.int8)
    w = rng.integers(-128, 128, ws, dtype=np.int8)
    sx = np.float32(0.017)
    sw = rng.uniform(0.001, 0.01, 20).astype(np.float32)
    acc = orc.convolution(x, w, orc.I8, (1, 1, 1))
    scale = np.broadcast_to((sx * sw).astype(np.float32).reshape(1, -1, 1, 1, 1), acc.shape)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.I32, orc.F32)
    got = ops.quant_convolution(dev(x), dev(w), (1, 1, 1), scale_x=dev(np.float32([sx])), scale_w=dev(sw))
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    got16 = ops.quant_convolution(dev(x), dev(w), (1, 1, 1), scale_x=dev(np.float32([sx])), scale_w=dev(sw),
                                  out_dtype=torch.float16)
    assert np.array_equal(half_bits(got16), orc.convert(want, orc.F32, orc.F16))
    # fp8: small integers are exact, and the float reference's known 3-D answer is met on operands
    # that fp8 represents exactly
    xi = rng.integers(-3, 4, xs).astype(np.float32)
    wi = rng.integers(-2, 3, ws).astype(np.float32)
    gotf = ops.quant_convolution(dev(orc.fp8_from_f32(xi)), dev(orc.fp8_from_f32(wi)), (1, 1, 1), fp8=True)
    assert gotf.dtype == torch.float32
    assert np.array_equal(gotf.cpu().numpy(), orc.convolution(xi, wi, orc.F32, (1, 1, 1)))


def test_fp8_convolution(ops):
    rng = np.random.default_rng(8)
    xs, ws = (2, 32, 10, 10), (24, 32, 3, 3)
    x = rng.standard_normal(xs).astype(np.float32)
    w = (rng.standard_normal(ws) * 0.05).astype(np.float32)
    xq = orc.quantizelinear(x.reshape(-1, xs[-1]), np.float32(np.abs(x).max() / 448), None, orc.F32,
                            orc.FP8).reshape(xs)
    wq = orc.quantizelinear(w.reshape(-1, ws[-1]), np.float32(np.abs(w).max() / 448), None, orc.F32,
                            orc.FP8).reshape(ws)
    want = orc.convolution(xq, wq, orc.FP8, (1, 1))
    got = ops.quant_convolution(dev(xq), dev(wq), (1, 1), fp8=True).cpu().numpy()
    # the fp8 matrix instructions keep about 20 bits below the largest product of a K-group
    mag = orc.convolution(np.abs(orc.fp8_to_f32(xq)).astype(np.float32),
                          np.abs(orc.fp8_to_f32(wq)).astype(np.float32), orc.F32, (1, 1))
    assert np.all(np.abs(got - want) <= np.maximum(1e-3 * np.abs(want), 2.0 ** -14 * mag))
    # small integers are exact
    xi = rng.integers(-3, 4, xs).astype(np.float32)
    wi = rng.integers(-2, 3, ws).astype(np.float32)
    got = ops.quant_convolution(dev(orc.fp8_from_f32(xi)), dev(orc.fp8_from_f32(wi)), (1, 1), fp8=True)
    assert np.array_equal(got.cpu().numpy(), orc.convolution(xi, wi, orc.F32, (1, 1)))


@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_fp8_direct_kernel_shapes_and_dequant_epilogue(ops, out):
    """fp8 through the direct kernel (16 | channels per group): two groups, a ragged channel tile, a K step whose
    second half is padding, row tiles over three images; scales applied as float(sum) * (scale_x * scale_w[o]),
    the fp8 GEMM's epilogue (quant_dot -> dequantizelinear, simplify_qdq.cpp:171-222)."""
    rng = np.random.default_rng(18)
    xs, ws = (3, 96, 9, 12), (80, 48, 3, 3)
    x = rng.standard_normal(xs).astype(np.float32)
    w = (rng.standard_normal(ws) * 0.05).astype(np.float32)
    sx = np.float32(np.abs(x).max() / 448)
    swt = np.float32(np.abs(w).max() / 448)
    xq = orc.quantizelinear(x.reshape(-1, xs[-1]), sx, None, orc.F32, orc.FP8).reshape(xs)
    wq = orc.quantizelinear(w.reshape(-1, ws[-1]), swt, None, orc.F32, orc.FP8).reshape(ws)
    acc = orc.convolution(xq, wq, orc.FP8, (1, 1), (1, 1), (1, 1), 2)
    mag = orc.convolution(np.abs(orc.fp8_to_f32(xq)).astype(np.float32),
                          np.abs(orc.fp8_to_f32(wq)).astype(np.float32), orc.F32, (1, 1), (1, 1), (1, 1), 2)
    bare = ops.quant_convolution(dev(xq), dev(wq), (1, 1), (1, 1), (1, 1), 2, fp8=True).cpu().numpy()
    assert np.all(np.abs(bare - acc) <= np.maximum(1e-3 * np.abs(acc), 2.0 ** -14 * mag))
    sw = (swt * rng.uniform(0.5, 2.0, 80)).astype(np.float32)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    got = ops.quant_convolution(dev(xq), dev(wq), (1, 1), (1, 1), (1, 1), 2, fp8=True, scale_x=dev(np.float32([sx])),
                                scale_w=dev(sw), out_dtype=td)
    # the kernel's own sums, scaled and converted as the reference does, are the result bit for bit
    scale = (sw * sx).astype(np.float32).reshape(1, -1, 1, 1)
    want = (bare * scale).astype(np.float32)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, orc.F16 if out == "f16" else orc.BF16))


def test_argument_errors(ops):
    x = dev(np.zeros((1, 4, 5, 5), np.int8))
    with pytest.raises(Exception):
        ops.quant_convolution(x, dev(np.zeros((2, 3, 3, 3), np.int8)))          # channels do not match
    with pytest.raises(Exception):
        ops.quant_convolution(x, dev(np.zeros((3, 2, 3, 3), np.int8)), group=2)  # O % group
    with pytest.raises(Exception):
        ops.quant_convolution(x, dev(np.zeros((2, 4, 3, 3), np.int8)), stride=(0, 1))
    with pytest.raises(Exception):
        ops.quant_convolution(x, dev(np.zeros((2, 4, 1, 3, 3), np.int8)))       # ranks differ
    with pytest.raises(Exception):
        ops.quant_convolution(dev(np.zeros((1, 4, 5, 5, 5), np.int8)), dev(np.zeros((2, 4, 3, 3, 3), np.int8)),
                              stride=(1, 1))                                      # two strides for three axes
    # a window larger than the padded input gives the minimum output size of one
    got = ops.quant_convolution(x, dev(np.ones((2, 4, 7, 7), np.int8)))
    assert tuple(got.shape) == (1, 2, 1, 1)


def test_caller_provided_result_and_workspace(ops):
    """The result and the workspace may be the caller's (reused from call to call): the same bits,
    written in place; a workspace that is too small or a result of the wrong shape is refused."""
    rng = np.random.default_rng(31)
    x = rng.integers(-128, 128, (2, 8, 9, 9), dtype=np.int8)
    w = rng.integers(-128, 128, (16, 8, 3, 3), dtype=np.int8)
    want = ops.quant_convolution(dev(x), dev(w), (1, 1))
    out = torch.full_like(want, -1)
    room = torch.empty(1 << 22, dtype=torch.uint8, device="cuda")
    got = ops.quant_convolution(dev(x), dev(w), (1, 1), out=out, workspace=room)
    assert got.data_ptr() == out.data_ptr() and torch.equal(out, want)
    with pytest.raises(Exception):
        ops.quant_convolution(dev(x), dev(w), (1, 1), workspace=torch.empty(8, dtype=torch.uint8, device="cuda"))
    with pytest.raises(Exception):
        ops.quant_convolution(dev(x), dev(w), (1, 1), out=torch.empty((2, 16, 9, 8), dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("xs,ws,group", [((2, 32, 12, 12), (24, 32, 3, 3), 1),      # direct kernel
                                         ((1, 20, 9, 9), (8, 10, 3, 3), 2)])       # gathered form (10 channels per group)
def test_fp8_nan_weight_on_zero_padded_forms(ops, xs, ws, group):
    """A NaN weight in an fp8 layer with padding.  The reference skips window elements outside the image, so
    the NaN spoils only outputs whose window has that element inside; the forms that work on a zero-padded
    copy (direct kernel, gathered form) also return NaN where the element falls on the border (0 * NaN).
    Pinned here: interior outputs agree with the oracle exactly, NaN included; border outputs are either the
    oracle's value or NaN, and every other output channel is untouched."""
    rng = np.random.default_rng(sum(xs) + sum(ws))
    xi = rng.integers(-3, 4, xs).astype(np.float32)
    wi = rng.integers(-2, 3, ws).astype(np.float32)
    wc = orc.fp8_from_f32(wi)
    wc[1, 0, 0, 0] = 0x7F
    wn = wi.copy()
    wn[1, 0, 0, 0] = np.nan
    got = ops.quant_convolution(dev(orc.fp8_from_f32(xi)), dev(wc), (1, 1), (1, 1), (1, 1), group, fp8=True).cpu().numpy()
    want = orc.convolution(xi, wn, orc.F32, (1, 1), (1, 1), (1, 1), group)
    assert np.isnan(want[:, 1, 1:, 1:]).all() and not np.isnan(want[:, 1, 0, :]).any()
    assert np.array_equal(got[:, :, 1:, 1:], want[:, :, 1:, 1:], equal_nan=True)
    others = [o for o in range(ws[0]) if o != 1]
    assert np.array_equal(got[:, others], want[:, others])
    border = got[:, 1, 0, :]
    assert (np.isnan(border) | (border == want[:, 1, 0, :])).all()
