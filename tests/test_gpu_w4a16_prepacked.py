"""GPU parity of the int4 weight-only GEMV over weights reordered ahead of time
(mi355_w4a16_prepack + mi355_w4a16_gemm_prepacked) against the CPU oracle's
unpack_int4 -> dequantizelinear -> dot chain and against mi355_w4a16_gemm."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev, half_dev, half_bits, ulp_distance_16

pytestmark = pytest.mark.gpu

G = 128


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def _case(rng, n, k, lo=0.005, hi=0.02):
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    scales = orc.half_from_f32(rng.uniform(lo, hi, (n, k // G)).astype(np.float32))
    a = orc.half_from_f32(rng.standard_normal((1, k)).astype(np.float32))
    return a, packed, scales, wq


# The tolerance of the int4 weight-only kernels: the reference sums exact fp16 products in double
# and rounds once; the kernel sums in fp32.  1e-3 relative, or 1 half ulp, or 2^-19 of sum|a||w|
# where the dot product cancels.
def _check(got_bits, want_bits, a, w_bits, identical=0.9):
    g = orc.half_to_f32(got_bits).astype(np.float64)
    w = orc.half_to_f32(want_bits).astype(np.float64)
    bound = np.abs(orc.half_to_f32(a)).astype(np.float64) @ \
        np.abs(orc.half_to_f32(w_bits)).astype(np.float64).T
    diff = np.abs(g - w)
    ok = (diff <= 1e-3 * np.abs(w)) | (ulp_distance_16(got_bits, want_bits) <= 1) | \
        (diff <= bound * 2.0**-19)
    assert ok.all(), ((~ok).sum(), diff.max())
    assert (got_bits == want_bits).mean() > identical


def _dequantized(wq, scales, zp):
    return orc.dequantizelinear(wq, np.repeat(scales, G, axis=1), np.full(wq.shape, zp, np.uint8),
                                orc.U8, orc.F16)


@pytest.mark.parametrize("n,k", [(16, 512), (64, 1024), (512, 4096), (272, 3584), (256, 14336), (48, 28672),
                                 (17600, 1536), (6160, 4096)])
@pytest.mark.parametrize("zp", [8, 0, 3])
def test_prepacked_gemv_matches_oracle(ops, n, k, zp):
    """Row groups x blocks of every launch shape: one block per wave, several blocks per wave,
    a block count that does not divide by the waves (7 blocks), several row groups per team
    (17600 rows), and the largest K; zero point 8 and 0 take the fused-multiply-add form, 3 the
    general one."""
    rng = np.random.default_rng(n + k + zp)
    a, packed, scales, wq = _case(rng, n, k)
    print("w4a16 prepacked", n, k, zp, flush=True)
    pk = ops.w4a16_prepack(dev(packed), half_dev(scales), G, zp=zp)
    assert pk is not None
    got = ops.w4a16_gemm_prepacked(half_dev(a), pk, n)
    want = orc.w4a16_matmul(a, packed, scales, zp, G)
    _check(half_bits(got), want, a, _dequantized(wq, scales, zp))
    # and next to the kernel that reads the operator's own layout
    other = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), G, zp=zp)
    _check(half_bits(got), half_bits(other), a, _dequantized(wq, scales, zp), identical=0.8)


@pytest.mark.parametrize("zp", [8, 4, 2, 1, 0, 5, 15])
@pytest.mark.parametrize("lo,hi", [(0.005, 0.02), (2.0**-10, 2.0**-9), (2.0**-5, 2.0**-4 - 2.0**-15), (2.0**-16, 2.0**-12),
                                   (0.5, 3.0), (-0.02, 0.02)])
def test_prepacked_dequantized_weights_are_exact(ops, zp, lo, hi):
    """With a one-hot activation row every output is one dequantized weight times +-1 or 2, so the
    nibble order of the reordered layout, the zero point, the scale lookup and the single
    truncation to half must match the reference bit for bit -- over both halves of the scale range
    the fused-multiply-add form takes, outside of it (subnormal-sized, large and negative scales:
    the general form), and for every kind of zero point."""
    rng = np.random.default_rng(int(zp * 1000 + abs(lo) * 1e6))
    n, k = 64, 1024
    _, packed, scales, wq = _case(rng, n, k, lo, hi)
    wdq = _dequantized(wq, scales, zp)
    pk = ops.w4a16_prepack(dev(packed), half_dev(scales), G, zp=zp)
    print("w4a16 prepacked exact", zp, lo, hi, flush=True)
    # every k-position class of the layout: all 32 offsets inside a lane's piece, each lane group,
    # each piece, both blocks
    ks = list(range(0, 32)) + [32 * i + 5 for i in range(1, 16)] + [512 + 97, 512 + 250, 1023]
    for kk in ks:
        a = np.zeros((1, k), np.float32)
        a[0, kk] = -2.0 if kk % 3 == 0 else 1.0
        ab = orc.half_from_f32(a)
        got = half_bits(ops.w4a16_gemm_prepacked(half_dev(ab), pk, n))
        want = orc.w4a16_matmul(ab, packed, scales, zp, G)
        # (the sign of a zero product is the sum's: +0 from the kernel's zero-initialised sum)
        nz = (want & 0x7fff) != 0
        assert np.array_equal(got[nz], want[nz]), (kk, np.flatnonzero(got != want)[:8])
        assert ((got[~nz] & 0x7fff) == 0).all()
        # the oracle's own dequantized weight, scaled by the one-hot value
        w1 = orc.half_to_f32(wdq[:, kk]) * a[0, kk]
        assert np.array_equal(orc.half_to_f32(got[0]), w1.astype(np.float32))


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 14336), (14336, 4096), (4096, 28672), (8192, 28672), (28672, 8192)])
def test_prepacked_full_size_config4_against_oracle(ops, k, n):
    """benchmark config 4 at its real sizes (M = 1) and the fused gate | up projection: sampled
    output columns against the oracle, every output against the kernel that reads the operator's
    layout.  (8192, 28672) has more row groups than one resident set of workgroups walks: one row
    group per workgroup in a grid larger than the device holds at once; (28672, 8192) is the largest K."""
    g = torch.Generator(device="cuda")
    g.manual_seed(k + n)
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda", generator=g)
    sc = (torch.rand((n, k // G), device="cuda", generator=g) * 0.015 + 0.005).half()
    x = torch.randn((1, k), device="cuda", generator=g).half()
    print("w4a16 prepacked full size", k, n, flush=True)
    pk = ops.w4a16_prepack(w, sc, G, zp=8)
    got = ops.w4a16_gemm_prepacked(x, pk, n)
    cols = sorted({0, 1, 15, 16, 17, 255, 256, n // 2 - 1, n // 2, n - 17, n - 16, n - 1} |
                  set(range(3, n, n // 41)))
    xh = half_bits(x)
    wc = w[cols].cpu().numpy()
    sb = half_bits(sc[cols])
    want = orc.w4a16_matmul(xh, wc, sb, 8, G)
    _check(half_bits(got[:, cols]), want, xh, _dequantized(orc.unpack_int4(wc), sb, 8))
    other = ops.w4a16_gemm(x, w, sc, G, zp=8)
    gb, ob = half_bits(got), half_bits(other)
    assert (ulp_distance_16(gb, ob) <= 1).mean() > 0.97
    assert np.abs(orc.half_to_f32(gb) - orc.half_to_f32(ob)).max() < 0.05


@pytest.mark.parametrize("m", [2, 5, 16])
@pytest.mark.parametrize("n,k", [(16, 512), (64, 1024), (512, 4096), (272, 3584), (6160, 4096), (14336, 4096)])
@pytest.mark.parametrize("zp", [8, 3])
def test_prepacked_rows_match_oracle(ops, m, n, k, zp):
    """2 .. 16 activation rows (each lane of the matrix-core operand its own row from the LDS),
    every launch shape of the one-row tests that fits the LDS, both dequantization forms; rows of
    a strided view."""
    if m * (2 * k + 16) + 256 + 16384 > 160 * 1024:
        pytest.skip("the rows do not fit the LDS")
    rng = np.random.default_rng(m * 7 + n + k + zp)
    _, packed, scales, wq = _case(rng, n, k)
    a = orc.half_from_f32(rng.standard_normal((m, k)).astype(np.float32))
    print("w4a16 prepacked rows", m, n, k, zp, flush=True)
    pk = ops.w4a16_prepack(dev(packed), half_dev(scales), G, zp=zp)
    got = ops.w4a16_gemm_prepacked(half_dev(a), pk, n)
    wdq = _dequantized(wq, scales, zp)
    if n * k <= 1 << 22:
        want = orc.w4a16_matmul(a, packed, scales, zp, G)
        _check(half_bits(got), want, a, wdq)
    else:       # the oracle on sampled columns
        cols = sorted(set(range(0, n, max(1, n // 97))) | {n - 1})
        want = orc.w4a16_matmul(a, packed[cols], scales[cols], zp, G)
        _check(half_bits(got)[:, cols], want, a, wdq[cols])
    other = ops.w4a16_gemm(half_dev(a), dev(packed), half_dev(scales), G, zp=zp)
    _check(half_bits(got), half_bits(other), a, wdq, identical=0.8)
    # every row equals the one-row product of that row (same kernel arithmetic, same order)
    for r in (0, m - 1):
        one = ops.w4a16_gemm_prepacked(half_dev(a[r:r + 1]), pk, n)
        assert np.array_equal(half_bits(one)[0], half_bits(got)[r])
    # rows 24 halves apart in memory, output rows wider than N
    wide = torch.zeros((m, k + 24), dtype=torch.float16, device="cuda")
    wide[:, :k] = half_dev(a)
    out = torch.zeros((m, n + 8), dtype=torch.float16, device="cuda")
    ops.w4a16_gemm_prepacked(wide[:, :k], pk, n, out=out[:, :n])
    assert np.array_equal(half_bits(out[:, :n]), half_bits(got)) and (out[:, n:] == 0).all()


def test_prepacked_rows_dequantized_weights_are_exact(ops):
    """one-hot activation rows, a different position per row: every output is one dequantized
    weight, bit for bit"""
    rng = np.random.default_rng(99)
    n, k, m = 64, 1024, 16
    _, packed, scales, wq = _case(rng, n, k)
    for zp in (8, 5):
        wdq = orc.half_to_f32(_dequantized(wq, scales, zp))
        pk = ops.w4a16_prepack(dev(packed), half_dev(scales), G, zp=zp)
        ks = rng.integers(0, k, m)
        a = np.zeros((m, k), np.float32)
        a[np.arange(m), ks] = 1.0
        got = orc.half_to_f32(half_bits(ops.w4a16_gemm_prepacked(half_dev(orc.half_from_f32(a)), pk, n)))
        assert np.array_equal(got, wdq[:, ks].T)


def test_prepacked_form_declines_other_shapes(ops):
    from amdmigraphx_amd import Mi355Error
    w = torch.zeros((24, 256), dtype=torch.uint8, device="cuda")          # N % 16 != 0
    s = torch.ones((24, 4), dtype=torch.float16, device="cuda")
    assert ops.w4a16_prepack(w, s, G) is None
    w = torch.zeros((32, 192), dtype=torch.uint8, device="cuda")          # K % 512 != 0
    s = torch.ones((32, 3), dtype=torch.float16, device="cuda")
    assert ops.w4a16_prepack(w, s, G) is None
    w = torch.zeros((32, 256), dtype=torch.uint8, device="cuda")          # group 64
    s = torch.ones((32, 8), dtype=torch.float16, device="cuda")
    assert ops.w4a16_prepack(w, s, 64) is None
    pk = ops.w4a16_prepack(w, torch.ones((32, 4), dtype=torch.float16, device="cuda"), G)
    with pytest.raises(Mi355Error):                                       # 17 rows: the other entry point's
        ops.w4a16_gemm_prepacked(torch.zeros((17, 512), dtype=torch.float16, device="cuda"), pk, 32)
    w = torch.zeros((32, 8192), dtype=torch.uint8, device="cuda")         # 16 rows of K = 16384: more than the LDS
    pk = ops.w4a16_prepack(w, torch.ones((32, 128), dtype=torch.float16, device="cuda"), G)
    with pytest.raises(Mi355Error):
        ops.w4a16_gemm_prepacked(torch.zeros((16, 16384), dtype=torch.float16, device="cuda"), pk, 32)
