"""GPU parity of the four-input quant_dot (block-scaled MX operands) against the CPU oracle.

Reference semantics (ref_quant_gemm::compute, src/targets/ref/lowering.cpp:221-242): float(a) *
scale_a and float(b) * scale_b element by element in float, then the float GEMM with a double
accumulator, one rounding to float.

Tolerance, stated up front.  With power-of-two block scales every scaled operand is exact, so the
reference result is the exact sum rounded once.  The block-scaled matrix-core instruction adds
the 128 products of a step in a fixed-point window and accumulates steps in fp32, exactly like the
fp8 instruction of the two-input quant_dot.  Required: equality where every partial sum is exactly
representable (small integers times powers of two); otherwise 1e-3 relative, or 2^-15 of
sum|a||b| where the sum cancels (the declared floor of the fp8 path).  Scales that are not block
constants or not powers of two take the exact path on the device: bit-exact."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def _fp4_values(packed):
    """[rows, K/2] packed e2m1 -> float32 [rows, K] the way unpack_fp4 + convert see them."""
    return orc.fp8_to_f32(orc.unpack_fp4(packed))


def _reference(a_f32, b_f32_nk, sa, sb):
    """the oracle's four-input form on full-size float operands and scales"""
    x = (a_f32.astype(np.float32) * sa.astype(np.float32)).astype(np.float32)
    w = (b_f32_nk.astype(np.float32) * sb.astype(np.float32)).astype(np.float32)
    return orc.gemm(x, np.swapaxes(w, -1, -2), orc.F32, orc.F32)


def _block_scales(rng, shape_rows, k, lo=-6, hi=6):
    e = rng.integers(lo, hi + 1, shape_rows + (k // 32,))
    return np.ldexp(np.float32(1.0), e).astype(np.float32)


def _close(got, want, a_abs, b_abs_nk, sa, sb):
    mag = (np.abs(a_abs) * sa).astype(np.float64) @ np.swapaxes((np.abs(b_abs_nk) * sb).astype(np.float64), -1, -2)
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    return (diff <= 1e-3 * np.abs(want)) | (diff <= mag * 2.0**-15)


def test_reference_known_answer_through_the_exact_path(ops, golden):
    """test/ref/dot_op.cpp:1836-1865 (quant_dot_4args_scales): scales alternate 0.5 / 1 inside a
    row, so no block is constant.  The operands 1..6 are fp8-representable; K = 3 is padded with
    zeros to one block of 32 for this entry point."""
    c = golden["quant_dot_4args_scales"]
    a = np.zeros((2, 32), np.float32)
    b = np.zeros((2, 32), np.float32)
    sa = np.ones((2, 32), np.float32)
    sb = np.ones((2, 32), np.float32)
    a[:, :3] = np.float32(c["a"]).reshape(2, 3)
    sa[:, :3] = np.float32(c["scale_a"]).reshape(2, 3)
    b[:, :3] = np.float32(c["b"]).reshape(3, 2).T
    sb[:, :3] = np.float32(c["scale_b"]).reshape(3, 2).T
    got = ops.quant_dot_mx(dev(orc.fp8_from_f32(a)), dev(orc.fp8_from_f32(b)), dev(sa), dev(sb))
    assert got.cpu().numpy().flatten().tolist() == c["gold"]


@pytest.mark.parametrize("m,n,k", [(16, 16, 128), (40, 24, 96), (130, 200, 512), (64, 64, 32), (257, 129, 1024)])
@pytest.mark.parametrize("a_fp4,b_fp4", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("compact", [False, True])
def test_block_scaled_matches_oracle(ops, m, n, k, a_fp4, b_fp4, compact):
    rng = np.random.default_rng(m * 3 + n + k + a_fp4 * 7 + b_fp4 * 11)
    print("mx", m, n, k, a_fp4, b_fp4, compact, flush=True)

    def operand(rows, fp4):
        if fp4:
            packed = rng.integers(0, 256, (rows, k // 2), dtype=np.uint8)
            return packed, _fp4_values(packed)
        codes = orc.fp8_from_f32(np.clip(rng.normal(0, 2.0, (rows, k)), -448, 448).astype(np.float32))
        return codes, orc.fp8_to_f32(codes)

    a_store, a_val = operand(m, a_fp4)
    b_store, b_val = operand(n, b_fp4)
    sa_c = _block_scales(rng, (m,), k)
    sb_c = _block_scales(rng, (n,), k)
    sa_full, sb_full = np.repeat(sa_c, 32, axis=1), np.repeat(sb_c, 32, axis=1)
    want = _reference(a_val, b_val, sa_full, sb_full)
    got = ops.quant_dot_mx(dev(a_store), dev(b_store), dev(sa_c if compact else sa_full),
                           dev(sb_c if compact else sb_full), a_fp4=a_fp4, b_fp4=b_fp4).cpu().numpy()
    ok = _close(got, want, a_val, b_val, sa_full, sb_full)
    mag = (np.abs(a_val) * sa_full).astype(np.float64) @ (np.abs(b_val) * sb_full).astype(np.float64).T
    worst = (np.abs(got.astype(np.float64) - want) / mag).max()
    assert ok.all(), ((~ok).sum(), np.abs(got - want).max(), "worst error / sum|a||b| = 2^%.1f" % np.log2(worst))
    if a_fp4 and b_fp4:
        # e2m1 products have two significant bits: most sums come out with the reference's bits
        assert (got == want).mean() > 0.5


def test_small_integer_operands_are_exact(ops):
    rng = np.random.default_rng(9)
    m, n, k = 96, 80, 256
    a = orc.fp8_from_f32(rng.integers(-4, 5, (m, k)).astype(np.float32))
    b = orc.fp8_from_f32(rng.integers(-4, 5, (n, k)).astype(np.float32))
    sa = _block_scales(rng, (m,), k, -2, 2)
    sb = _block_scales(rng, (n,), k, -2, 2)
    want = _reference(orc.fp8_to_f32(a), orc.fp8_to_f32(b), np.repeat(sa, 32, 1), np.repeat(sb, 32, 1))
    got = ops.quant_dot_mx(dev(a), dev(b), dev(sa), dev(sb)).cpu().numpy()
    assert np.array_equal(got, want)


def test_batched(ops):
    rng = np.random.default_rng(10)
    bt, m, n, k = 3, 40, 24, 96
    pa = rng.integers(0, 256, (bt, m, k // 2), dtype=np.uint8)
    pb = rng.integers(0, 256, (bt, n, k // 2), dtype=np.uint8)
    sa = _block_scales(rng, (bt, m), k, -1, 1)     # products within 2^7 of each other: exact sums
    sb = _block_scales(rng, (bt, n), k, -1, 1)
    want = _reference(_fp4_values(pa.reshape(-1, k // 2)).reshape(bt, m, k),
                      _fp4_values(pb.reshape(-1, k // 2)).reshape(bt, n, k),
                      np.repeat(sa, 32, axis=2), np.repeat(sb, 32, axis=2))
    got = ops.quant_dot_mx(dev(pa), dev(pb), dev(sa), dev(sb), a_fp4=True, b_fp4=True).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("fp4,bt,m,n,k", [
    (True, 1, 300, 520, 128), (True, 1, 257, 260, 384), (True, 2, 130, 300, 640), (True, 1, 512, 256, 2048),
    (False, 1, 300, 520, 64), (False, 1, 257, 260, 192), (False, 2, 130, 300, 320), (False, 1, 512, 256, 1024)])
def test_staged_kernel_exact_sums(ops, fp4, bt, m, n, k):
    """Packed fp4 x fp4 with K % 128 == 0 and fp8 x fp8 with K % 64 == 0 run on the LDS-staged
    kernel (256 x 256 tiles, 64-byte slabs: one, three, five and many of them; several tiles with
    ragged edges; batches).  Operands and scales are chosen so that every partial sum is exact in
    fp32 (small codes, scales within a factor of four), so each output must carry the reference's
    bits: a misplaced chunk, slab, tile or exponent byte shows."""
    rng = np.random.default_rng(m + 3 * n + 7 * k + bt)
    if fp4:
        # codes of magnitude 0, 0.5, 1, 1.5 with either sign
        pa = rng.integers(0, 4, (bt, m, k // 2), dtype=np.uint8) | (rng.integers(0, 4, (bt, m, k // 2), dtype=np.uint8) << 4)
        pb = rng.integers(0, 4, (bt, n, k // 2), dtype=np.uint8) | (rng.integers(0, 4, (bt, n, k // 2), dtype=np.uint8) << 4)
        pa |= rng.integers(0, 2, pa.shape, dtype=np.uint8) << 3
        pb |= rng.integers(0, 2, pb.shape, dtype=np.uint8) << 7
        av = _fp4_values(pa.reshape(-1, k // 2)).reshape(bt, m, k)
        bv = _fp4_values(pb.reshape(-1, k // 2)).reshape(bt, n, k)
    else:
        pa = orc.fp8_from_f32(rng.integers(-4, 5, (bt, m, k)).astype(np.float32))
        pb = orc.fp8_from_f32(rng.integers(-4, 5, (bt, n, k)).astype(np.float32))
        av, bv = orc.fp8_to_f32(pa), orc.fp8_to_f32(pb)
    sa = _block_scales(rng, (bt, m), k, -1, 1)
    sb = _block_scales(rng, (bt, n), k, -1, 1)
    want = _reference(av, bv, np.repeat(sa, 32, axis=2), np.repeat(sb, 32, axis=2))
    print("mx staged", fp4, bt, m, n, k, flush=True)
    got = ops.quant_dot_mx(dev(pa), dev(pb), dev(sa), dev(sb), a_fp4=fp4, b_fp4=fp4).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("bt,m,n,k", [(1, 300, 520, 4096), (2, 257, 260, 4352), (1, 512, 256, 4224), (1, 130, 300, 8192),
                                      (1, 600, 256, 5120)])
def test_four_wave_fp4_kernel_exact_sums(ops, bt, m, n, k):
    """Packed fp4 x fp4 with K >= 4096: the four-wave kernel (exponent words loaded per lane, two scaled
    MFMAs per tile pair and slab).  Even and odd slab counts, batches, ragged tiles; sums exact in fp32 as in
    test_staged_kernel_exact_sums, so every output carries the reference's bits."""
    rng = np.random.default_rng(m + 3 * n + 7 * k + bt)
    pa = rng.integers(0, 4, (bt, m, k // 2), dtype=np.uint8) | (rng.integers(0, 4, (bt, m, k // 2), dtype=np.uint8) << 4)
    pb = rng.integers(0, 4, (bt, n, k // 2), dtype=np.uint8) | (rng.integers(0, 4, (bt, n, k // 2), dtype=np.uint8) << 4)
    pa |= rng.integers(0, 2, pa.shape, dtype=np.uint8) << 3
    pb |= rng.integers(0, 2, pb.shape, dtype=np.uint8) << 7
    av = _fp4_values(pa.reshape(-1, k // 2)).reshape(bt, m, k)
    bv = _fp4_values(pb.reshape(-1, k // 2)).reshape(bt, n, k)
    sa = _block_scales(rng, (bt, m), k, -1, 1)
    sb = _block_scales(rng, (bt, n), k, -1, 1)
    want = _reference(av, bv, np.repeat(sa, 32, axis=2), np.repeat(sb, 32, axis=2))
    print("mx four-wave fp4", bt, m, n, k, flush=True)
    got = ops.quant_dot_mx(dev(pa), dev(pb), dev(sa), dev(sb), a_fp4=True, b_fp4=True).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("bt,m,n,k", [(1, 300, 520, 2048), (2, 257, 260, 2176), (1, 512, 256, 2112), (1, 130, 300, 4096)])
def test_four_wave_fp8_kernel_exact_sums(ops, bt, m, n, k):
    """fp8 x fp8 with K >= 2048: the four-wave kernel (one scaled MFMA per tile pair and slab, byte g of the
    row's exponent word for lane group g).  Even and odd slab counts, batches, ragged tiles; exact sums."""
    rng = np.random.default_rng(m + 3 * n + 7 * k + bt)
    pa = orc.fp8_from_f32(rng.integers(-4, 5, (bt, m, k)).astype(np.float32))
    pb = orc.fp8_from_f32(rng.integers(-4, 5, (bt, n, k)).astype(np.float32))
    av, bv = orc.fp8_to_f32(pa), orc.fp8_to_f32(pb)
    sa = _block_scales(rng, (bt, m), k, -1, 1)
    sb = _block_scales(rng, (bt, n), k, -1, 1)
    want = _reference(av, bv, np.repeat(sa, 32, axis=2), np.repeat(sb, 32, axis=2))
    print("mx four-wave fp8", bt, m, n, k, flush=True)
    got = ops.quant_dot_mx(dev(pa), dev(pb), dev(sa), dev(sb), a_fp4=False, b_fp4=False).cpu().numpy()
    assert np.array_equal(got, want)


def test_four_wave_fp4_kernel_full_range_operands(ops):
    """The same kernel on codes and exponents over their whole range: the path's tolerance."""
    rng = np.random.default_rng(23)
    m, n, k = 384, 512, 4096
    pa = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    pb = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    av, bv = _fp4_values(pa), _fp4_values(pb)
    sa_c, sb_c = _block_scales(rng, (m,), k), _block_scales(rng, (n,), k)
    sa, sb = np.repeat(sa_c, 32, axis=1), np.repeat(sb_c, 32, axis=1)
    want = _reference(av, bv, sa, sb)
    got = ops.quant_dot_mx(dev(pa), dev(pb), dev(sa_c), dev(sb_c), a_fp4=True, b_fp4=True).cpu().numpy()
    assert _close(got, want, av, bv, sa, sb).all()


def test_staged_kernel_full_range_operands(ops):
    """The staged kernel on operands and exponents over their whole range: the path's tolerance."""
    rng = np.random.default_rng(21)
    m, n, k = 384, 512, 1024
    pa = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    pb = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    av, bv = _fp4_values(pa), _fp4_values(pb)
    sa_c, sb_c = _block_scales(rng, (m,), k), _block_scales(rng, (n,), k)
    sa, sb = np.repeat(sa_c, 32, axis=1), np.repeat(sb_c, 32, axis=1)
    want = _reference(av, bv, sa, sb)
    got = ops.quant_dot_mx(dev(pa), dev(pb), dev(sa_c), dev(sb_c), a_fp4=True, b_fp4=True).cpu().numpy()
    assert _close(got, want, av, bv, sa, sb).all()


@pytest.mark.parametrize("kind", ["not_a_power_of_two", "varies_inside_a_block", "negative", "zero"])
def test_general_scales_take_the_exact_path(ops, kind):
    """Scales the instruction cannot take are found on the device; the result is then the
    operator's own arithmetic, bit for bit."""
    rng = np.random.default_rng(11)
    m, n, k = 33, 20, 64
    pa = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    b = orc.fp8_from_f32(rng.normal(0, 1.0, (n, k)).astype(np.float32))
    sa = np.repeat(_block_scales(rng, (m,), k), 32, axis=1)
    sb = np.repeat(_block_scales(rng, (n,), k), 32, axis=1)
    if kind == "not_a_power_of_two":
        sb[5, 32:] = 0.3
    elif kind == "varies_inside_a_block":
        sa[7, 40] *= 2
    elif kind == "negative":
        sa[0, :32] = -0.5
    else:
        sb[3, :32] = 0.0
    want = _reference(_fp4_values(pa), orc.fp8_to_f32(b), sa, sb)
    got = ops.quant_dot_mx(dev(pa), dev(b), dev(sa), dev(sb), a_fp4=True).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_good_scales_after_flagged_ones_in_one_workspace(ops):
    """The workspace word that marks "this call's scales need the exact path" is never cleared; every
    eager call writes and compares its own number.  A call with power-of-two scales that follows a
    flagged call in the same workspace must therefore be back on the matrix cores: it gives the bits
    of the same call in a fresh workspace (the exact path would give the oracle's bits instead, which
    differ from the matrix cores' in the last places on these operands)."""
    rng = np.random.default_rng(12)
    m, n, k = 96, 80, 512
    a = orc.fp8_from_f32(rng.normal(0, 1.0, (m, k)).astype(np.float32))
    b = orc.fp8_from_f32(rng.normal(0, 1.0, (n, k)).astype(np.float32))
    sa, sb = _block_scales(rng, (m,), k), _block_scales(rng, (n,), k)
    bad = sb.copy()
    bad[3, 1] = 0.3
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    fresh = ops.quant_dot_mx(dev(a), dev(b), dev(sa), dev(sb)).cpu().numpy()
    exact = ops.quant_dot_mx(dev(a), dev(b), dev(sa), dev(bad), workspace=ws).cpu().numpy()
    want_bad = _reference(orc.fp8_to_f32(a), orc.fp8_to_f32(b), np.repeat(sa, 32, axis=1), np.repeat(bad, 32, axis=1))
    assert np.array_equal(exact.view(np.uint32), want_bad.view(np.uint32))
    again = ops.quant_dot_mx(dev(a), dev(b), dev(sa), dev(sb), workspace=ws).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), fresh.view(np.uint32))
    want = _reference(orc.fp8_to_f32(a), orc.fp8_to_f32(b), np.repeat(sa, 32, axis=1), np.repeat(sb, 32, axis=1))
    assert not np.array_equal(fresh.view(np.uint32), want.view(np.uint32)), "operands too tame to tell the paths apart"


def test_argument_errors(ops):
    from amdmigraphx_amd import Mi355Error
    a = torch.zeros((4, 48), dtype=torch.uint8, device="cuda")      # K = 48: not whole blocks
    s = torch.ones((4, 48), device="cuda")
    with pytest.raises(Mi355Error):
        ops.quant_dot_mx(a, a, s, s)
