"""GPU parity of the int4 weight-only GEMM / GEMV against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev, half_dev, half_bits, ulp_distance_16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def _case(rng, m, n, k, g):
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    scales = orc.half_from_f32(rng.uniform(0.005, 0.02, (n, k // g)).astype(np.float32))
    a = orc.half_from_f32(rng.standard_normal((m, k)).astype(np.float32))
    return a, packed, scales, wq


# Tolerance: the reference sums exact fp16 products in double and rounds once
# (to float, then truncates to half); the kernel sums in fp32.  An output
# passes within 1e-3 relative, or 1 half ulp, or 2^-19 of sum|a||w| where the
# dot product cancels.
def _check(got_bits, want_bits, a, w_bits):
    g = orc.half_to_f32(got_bits).astype(np.float64)
    w = orc.half_to_f32(want_bits).astype(np.float64)
    bound = np.abs(orc.half_to_f32(a)).astype(np.float64) @ \
        np.abs(orc.half_to_f32(w_bits)).astype(np.float64).T
    diff = np.abs(g - w)
    ok = (diff <= 1e-3 * np.abs(w)) | (ulp_distance_16(got_bits, want_bits) <= 1) | \
        (diff <= bound * 2.0**-19)
    assert ok.all(), ((~ok).sum(), diff.max())
    assert (got_bits == want_bits).mean() > 0.9


@pytest.mark.parametrize("m", [1, 2, 3, 16])
@pytest.mark.parametrize("n,k", [(64, 256), (512, 4096), (100, 2048 + 128), (256, 14336)])
def test_w4a16_matches_oracle(ops, m, n, k):
    rng = np.random.default_rng(m * 100 + n + k)
    g = 128
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    got = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8)
    sf = np.repeat(scales, g, axis=1)
    wdq = orc.dequantizelinear(wq, sf, np.full(wq.shape, 8, np.uint8), orc.U8, orc.F16)
    _check(half_bits(got), want, a, wdq)


def test_w4a16_group_zero_points_and_group32(ops):
    rng = np.random.default_rng(9)
    m, n, k, g = 2, 96, 1024, 32
    a, packed, scales, wq = _case(rng, m, n, k, g)
    zp = rng.integers(0, 16, (n, k // g), dtype=np.uint8)
    want = orc.w4a16_matmul(a, packed, scales, zp, g)
    got = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=dev(zp))
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.repeat(zp, g, axis=1),
                               orc.U8, orc.F16)
    _check(half_bits(got), want, a, wdq)
    # the same zero points packed two per byte (MatMulNBits input layout)
    zpp = orc.pack_int4(zp)
    got = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=dev(zpp),
                         zp_mode=ops.W4ZP.PACKED)
    _check(half_bits(got), want, a, wdq)


def test_w4a16_dequantized_weights_are_exact(ops):
    """With one-hot activations the output is a single dequantized weight, so
    the unpack order, zero point, scale lookup and the truncating half
    conversions must all match bit for bit."""
    rng = np.random.default_rng(10)
    n, k, g = 128, 512, 128
    _, packed, scales, wq = _case(rng, 1, n, k, g)
    a = np.zeros((4, k), np.float32)
    for i, kk in enumerate((0, 1, 255, 511)):
        a[i, kk] = 1.0
    ab = orc.half_from_f32(a)
    want = orc.w4a16_matmul(ab, packed, scales, 8, g)
    got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=8)
    assert np.array_equal(half_bits(got), want)
