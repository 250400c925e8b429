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


# ---- M >= 2: matrix-core kernel (N % 16 == 0, K % 128 == 0) ---------------------------

@pytest.mark.parametrize("m", [2, 16, 17, 40, 128, 150])
@pytest.mark.parametrize("n,k,g", [(64, 256, 128), (256, 4096, 128), (48, 1152, 64), (32, 14336, 128)])
def test_w4a16_matrix_core_kernel_matches_oracle(ops, m, n, k, g):
    rng = np.random.default_rng(m * 7 + n + k)
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    print("w4a16 mfma", m, n, k, g, flush=True)
    got = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8)
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8),
                               orc.U8, orc.F16)
    _check(half_bits(got), want, a, wdq)


def test_w4a16_matrix_core_kernel_exact_weights_all_zero_point_forms(ops):
    """One-hot activations in every row of a 16-row tile and in a second tile: each
    output is one dequantized weight and must match bit for bit, for scalar,
    per-group and packed zero points, and for scales too small for the
    (s, s/16) form of the dequantization."""
    rng = np.random.default_rng(12)
    n, k, g = 64, 512, 32
    m = 24
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    a = np.zeros((m, k), np.float32)
    for i in range(m):
        a[i, (i * 37 + 5) % k] = 1.0 if i % 2 == 0 else -2.0
    ab = orc.half_from_f32(a)
    for lo, hi in ((0.005, 0.02), (2.0**-16, 2.0**-12), (0.5, 3.0)):
        scales = orc.half_from_f32(rng.uniform(lo, hi, (n, k // g)).astype(np.float32))
        zp = rng.integers(0, 16, (n, k // g), dtype=np.uint8)
        for zmode in ("scalar", "group", "packed"):
            print("w4a16 mfma exact", lo, zmode, flush=True)
            if zmode == "scalar":
                want = orc.w4a16_matmul(ab, packed, scales, 3, g)
                got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=3)
            elif zmode == "group":
                want = orc.w4a16_matmul(ab, packed, scales, zp, g)
                got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=dev(zp))
            else:
                want = orc.w4a16_matmul(ab, packed, scales, zp, g)
                got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g,
                                     zp=dev(orc.pack_int4(zp)), zp_mode=ops.W4ZP.PACKED)
            assert np.array_equal(half_bits(got), want), (lo, zmode)


# ---- more than 32 rows and N % 128 == 0: the 64 x 128 tile kernel ------------------------

@pytest.mark.parametrize("m,n,k,g", [(33, 128, 128, 128), (64, 256, 384, 128), (65, 128, 1152, 64),
                                     (100, 384, 2048 + 128, 32), (128, 128, 512, 128), (300, 256, 640, 128),
                                     (129, 128, 384, 64)])
def test_w4a16_tile_kernel_matches_oracle(ops, m, n, k, g):
    """K an even and an odd multiple of 128 (the last chunk of 256 is then half used), row
    counts that leave the second 64-row block nearly empty, several groups per step."""
    rng = np.random.default_rng(m * 11 + n + k + g)
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    print("w4a16 tile", m, n, k, g, flush=True)
    got = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8)
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8),
                               orc.U8, orc.F16)
    _check(half_bits(got), want, a, wdq)


def test_w4a16_tile_kernel_exact_weights_all_zero_point_forms(ops):
    """One-hot activations in 70 rows (both 64-row blocks): each output is one dequantized
    weight and must match bit for bit, for scalar, per-group and packed zero points and
    for scales on both sides of the range of the (s, s/16) form."""
    rng = np.random.default_rng(21)
    n, k, g = 256, 640, 32
    m = 70
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    a = np.zeros((m, k), np.float32)
    for i in range(m):
        a[i, (i * 53 + 7) % k] = 1.0 if i % 2 == 0 else -2.0
    ab = orc.half_from_f32(a)
    for lo, hi in ((0.005, 0.02), (2.0**-16, 2.0**-12), (0.5, 3.0)):
        scales = orc.half_from_f32(rng.uniform(lo, hi, (n, k // g)).astype(np.float32))
        zp = rng.integers(0, 16, (n, k // g), dtype=np.uint8)
        for zmode in ("scalar", "group", "packed"):
            print("w4a16 tile exact", lo, zmode, flush=True)
            if zmode == "scalar":
                want = orc.w4a16_matmul(ab, packed, scales, 3, g)
                got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=3)
            elif zmode == "group":
                want = orc.w4a16_matmul(ab, packed, scales, zp, g)
                got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=dev(zp))
            else:
                want = orc.w4a16_matmul(ab, packed, scales, zp, g)
                got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g,
                                     zp=dev(orc.pack_int4(zp)), zp_mode=ops.W4ZP.PACKED)
            assert np.array_equal(half_bits(got), want), (lo, zmode)


def test_w4a16_tile_kernel_strided_activations_and_output(ops):
    rng = np.random.default_rng(22)
    m, n, k, g = 90, 128, 384, 128
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    big = np.zeros((m, k + 64), np.uint16)
    big[:, :k] = a
    a_dev = half_dev(big)[:, :k]
    out = torch.zeros((m, n + 16), dtype=torch.float16, device="cuda")
    ops.w4a16_gemm(a_dev, dev(packed), half_dev(scales), g, zp=8, out=out[:, :n])
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8),
                               orc.U8, orc.F16)
    _check(half_bits(out[:, :n].contiguous()), want, a, wdq)
    assert (out[:, n:] == 0).all()


def test_w4a16_matrix_core_kernel_strided_activations_and_output(ops):
    rng = np.random.default_rng(13)
    m, n, k, g = 20, 80, 384, 128
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    big = np.zeros((m, k + 64), np.uint16)
    big[:, :k] = a
    a_dev = half_dev(big)[:, :k]
    out = torch.zeros((m, n + 16), dtype=torch.float16, device="cuda")
    ops.w4a16_gemm(a_dev, dev(packed), half_dev(scales), g, zp=8, out=out[:, :n])
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8),
                               orc.U8, orc.F16)
    _check(half_bits(out[:, :n].contiguous()), want, a, wdq)
    assert (out[:, n:] == 0).all()


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 14336), (14336, 4096)])
def test_w4a16_full_size_config4_shapes(ops, k, n):
    """benchmark config 4 at its real sizes, M in {1, 16, 128}: one-hot activation rows pick
    single dequantized weights out of the full matrix (exact, for every kernel), and the
    batched kernels agree with the M = 1 kernel row by row within the summation tolerance."""
    g = 128
    gen = torch.Generator(device="cuda")
    gen.manual_seed(k * 3 + n)
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda", generator=gen)
    sc = (torch.rand((n, k // g), device="cuda", generator=gen) * 0.015 + 0.005).half()
    print("w4a16 full size", k, n, flush=True)
    # expected dequantized weights for a few k positions, computed with torch on the device:
    # half((q - 8) * scale) with truncation = the float product's bits shifted
    ks = [0, 1, 127, 128, k // 2 + 5, k - 1]
    onehot = torch.zeros((len(ks), k), dtype=torch.float16, device="cuda")
    for i, kk in enumerate(ks):
        onehot[i, kk] = 1.0
    want_rows = []
    for kk in ks:
        byte = w[:, kk // 2].int()
        q = (byte >> 4) if kk % 2 else (byte & 0xF)
        prod = (q - 8).float() * sc[:, kk // g].float()
        want_rows.append(orc.half_from_f32(prod.cpu().numpy()))
    want = np.stack(want_rows)
    for m in (1, 16, 128):
        a = torch.zeros((m, k), dtype=torch.float16, device="cuda")
        rows = min(m, len(ks))
        a[:rows] = onehot[:rows]
        got = ops.w4a16_gemm(a, w, sc, g, zp=8)
        assert np.array_equal(half_bits(got[:rows]), want[:rows]), m
        assert (got[rows:] == 0).all()
    # random activations: every row of the M = 16 / 128 result against the M = 1 kernel
    x = torch.randn((128, k), device="cuda", generator=gen).half()
    big = ops.w4a16_gemm(x, w, sc, g, zp=8)
    mid = ops.w4a16_gemm(x[:16], w, sc, g, zp=8)
    for r in (0, 7, 15):
        one = ops.w4a16_gemm(x[r:r + 1], w, sc, g, zp=8)
        for other in (big[r:r + 1], mid[r:r + 1]):
            d = (other.float() - one.float()).abs()
            tol = torch.maximum(one.float().abs() * 2e-3, torch.tensor(2e-3, device="cuda"))
            assert (d <= tol).all(), (r, d.max().item())


@pytest.mark.parametrize("m", [1, 16, 128])
@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 14336), (14336, 4096)])
def test_w4a16_full_size_config4_against_oracle(ops, m, k, n):
    """benchmark config 4 at its real sizes: sampled output columns (weight rows) of the full
    product against the oracle's unpack_int4 -> dequantizelinear -> dot chain, for the bare call
    and the call with a workspace."""
    g = 128
    gen = torch.Generator(device="cuda")
    gen.manual_seed(k * 5 + n + m)
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda", generator=gen)
    sc = (torch.rand((n, k // g), device="cuda", generator=gen) * 0.015 + 0.005).half()
    x = torch.randn((m, k), device="cuda", generator=gen).half()
    print("w4a16 full size vs oracle", m, k, n, flush=True)
    cols = sorted(set(list(range(0, 16)) + [127, 128, 129, n // 2 - 1, n // 2, n - 130, n - 17, n - 16, n - 2, n - 1]
                      + list(range(1000, 1032))))
    a = half_bits(x)
    packed = w[cols].cpu().numpy()
    scales = half_bits(sc[cols])
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    wq = orc.unpack_int4(packed)
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8), orc.U8, orc.F16)
    got = ops.w4a16_gemm(x, w, sc, g, zp=8)
    _check(half_bits(got[:, cols]), want, a, wdq)
    nbytes = ops.w4a16_gemm_workspace_size(m, n, k, g)
    if nbytes > 0:
        ws = torch.full((nbytes,), 0x7F, dtype=torch.uint8, device="cuda")
        got = ops.w4a16_gemm(x, w, sc, g, zp=8, workspace=ws)
        _check(half_bits(got[:, cols]), want, a, wdq)


# ---- the tile kernel with a workspace: K split over more workgroups --------------------------

@pytest.mark.parametrize("m,n,k,g", [(64, 256, 1152, 64), (100, 384, 2048 + 128, 32), (130, 128, 1024, 128),
                                     (128, 512, 4096, 128), (40, 128, 1536, 128), (300, 256, 1152, 64)])
def test_w4a16_tile_kernel_split_k_with_workspace(ops, m, n, k, g):
    """Shares of K leave float partial sums in the workspace, a second kernel adds them in a fixed
    order: the oracle's value within the path's tolerance, the same bits on every call; K an odd
    multiple of 128, shares of unequal length, more than 128 rows."""
    rng = np.random.default_rng(m * 7 + n + k + g)
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    nbytes = ops.w4a16_gemm_workspace_size(m, n, k, g)
    assert nbytes > 0
    ws = torch.full((nbytes,), 0x7F, dtype=torch.uint8, device="cuda")
    print("w4a16 tile workspace", m, n, k, g, nbytes, flush=True)
    out = torch.zeros((m, n + 8), dtype=torch.float16, device="cuda")
    ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8, out=out[:, :n], workspace=ws)
    got = out[:, :n].contiguous()
    again = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8, workspace=ws)
    assert torch.equal(got.view(torch.int16), again.view(torch.int16))
    assert (out[:, n:] == 0).all()
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8),
                               orc.U8, orc.F16)
    _check(half_bits(got), want, a, wdq)
    # a workspace that is too small is not an error
    small = torch.empty(256, dtype=torch.uint8, device="cuda")
    one_pass = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8)
    assert torch.equal(ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8,
                                      workspace=small).view(torch.int16), one_pass.view(torch.int16))


def test_w4a16_tile_kernel_split_k_exact_weights(ops):
    """One-hot activations: every partial sum is one dequantized weight or zero, so the split
    result must match the oracle bit for bit, for the three zero-point forms."""
    rng = np.random.default_rng(23)
    n, k, g, m = 256, 1280, 32, 70
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    a = np.zeros((m, k), np.float32)
    for i in range(m):
        a[i, (i * 53 + 7) % k] = 1.0 if i % 2 == 0 else -2.0
    ab = orc.half_from_f32(a)
    scales = orc.half_from_f32(rng.uniform(0.005, 0.02, (n, k // g)).astype(np.float32))
    zp = rng.integers(0, 16, (n, k // g), dtype=np.uint8)
    nbytes = ops.w4a16_gemm_workspace_size(m, n, k, g)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    for zmode in ("scalar", "group", "packed"):
        print("w4a16 tile workspace exact", zmode, flush=True)
        if zmode == "scalar":
            want = orc.w4a16_matmul(ab, packed, scales, 3, g)
            got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=3, workspace=ws)
        elif zmode == "group":
            want = orc.w4a16_matmul(ab, packed, scales, zp, g)
            got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=dev(zp), workspace=ws)
        else:
            want = orc.w4a16_matmul(ab, packed, scales, zp, g)
            got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g,
                                 zp=dev(orc.pack_int4(zp)), zp_mode=ops.W4ZP.PACKED, workspace=ws)
        assert np.array_equal(half_bits(got), want), zmode


# ---- the matrix-core kernel for few rows with a workspace: widest column tile, K split ----------

@pytest.mark.parametrize("m,n,k,g", [(16, 256, 8192, 128), (2, 64, 8192 + 128, 64), (17, 320, 8192, 128),
                                     (40, 96, 16384 + 128, 32), (48, 160, 16384 + 128, 128),
                                     (32, 1024, 14336, 128)])
def test_w4a16_matrix_core_kernel_split_k_with_workspace(ops, m, n, k, g):
    rng = np.random.default_rng(m * 5 + n + k + g)
    a, packed, scales, wq = _case(rng, m, n, k, g)
    want = orc.w4a16_matmul(a, packed, scales, 8, g)
    nbytes = ops.w4a16_gemm_workspace_size(m, n, k, g)
    assert nbytes > 0
    ws = torch.full((nbytes,), 0x7F, dtype=torch.uint8, device="cuda")
    print("w4a16 mfma workspace", m, n, k, g, nbytes, flush=True)
    out = torch.zeros((m, n + 8), dtype=torch.float16, device="cuda")
    ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8, out=out[:, :n], workspace=ws)
    got = out[:, :n].contiguous()
    again = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), g, zp=8, workspace=ws)
    assert torch.equal(got.view(torch.int16), again.view(torch.int16))
    assert (out[:, n:] == 0).all()
    wdq = orc.dequantizelinear(wq, np.repeat(scales, g, axis=1), np.full(wq.shape, 8, np.uint8),
                               orc.U8, orc.F16)
    _check(half_bits(got), want, a, wdq)


def test_w4a16_matrix_core_kernel_split_k_exact_weights(ops):
    """One-hot activations, the three zero-point forms: bit for bit the oracle's weights."""
    rng = np.random.default_rng(24)
    n, k, g, m = 128, 8192, 32, 12
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    a = np.zeros((m, k), np.float32)
    for i in range(m):
        a[i, (i * 531 + 7) % k] = 1.0 if i % 2 == 0 else -2.0
    ab = orc.half_from_f32(a)
    scales = orc.half_from_f32(rng.uniform(0.005, 0.02, (n, k // g)).astype(np.float32))
    zp = rng.integers(0, 16, (n, k // g), dtype=np.uint8)
    nbytes = ops.w4a16_gemm_workspace_size(m, n, k, g)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    for zmode in ("scalar", "group", "packed"):
        print("w4a16 mfma workspace exact", zmode, flush=True)
        if zmode == "scalar":
            want = orc.w4a16_matmul(ab, packed, scales, 3, g)
            got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=3, workspace=ws)
        elif zmode == "group":
            want = orc.w4a16_matmul(ab, packed, scales, zp, g)
            got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g, zp=dev(zp), workspace=ws)
        else:
            want = orc.w4a16_matmul(ab, packed, scales, zp, g)
            got = ops.w4a16_gemm(half_dev(ab), dev(packed), half_dev(scales), g,
                                 zp=dev(orc.pack_int4(zp)), zp_mode=ops.W4ZP.PACKED, workspace=ws)
        assert np.array_equal(half_bits(got), want), zmode
