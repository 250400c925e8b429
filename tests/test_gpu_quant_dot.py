"""GPU parity of quant_dot (+ fused dequantizelinear) against the CPU oracle,
through the C ABI.  int32 accumulators and every int8-path output are required
bit-exact; fp8 outputs within the stated floating-point tolerance."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev, bf16_bits, half_bits, ulp_distance_16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def _iota(lens, dtype, start=0):
    n = int(np.prod(lens))
    return (np.arange(n, dtype=np.int64) + start).astype(dtype).reshape(lens)


def test_reference_known_answers_on_gpu(ops, golden):
    """The 15 quant_dot cases of test/ref/dot_op.cpp run through the library
    (transposed views and batches exercise the any-stride kernel)."""
    for c in golden["quant_dot"]:
        a = _iota(c["a"]["lens"], np.int8)
        b = _iota(c["b"]["lens"], np.int8)
        ta, tb = dev(a), dev(b)
        if c["alpha"] != 1:
            af = (np.float32(c["alpha"]) * a.astype(np.float32))
            ta = dev(orc.convert(af, orc.F32, orc.I8).reshape(a.shape))
        if c["a_perm"]:
            ta = ta.permute(c["a_perm"])
        if c["b_perm"]:
            tb = tb.permute(c["b_perm"])
        out = ops.quant_dot(ta, tb).cpu().numpy().astype(np.int64)
        if c["uses_c"] and c["beta"] != 0:
            cm = _iota(c["c"]["lens"], np.int32, c["iota_start"]["c"])
            out = out + orc.convert(cm.astype(np.float32) * np.float32(c["beta"]),
                                    orc.F32, orc.I32).reshape(out.shape)
        assert out.flatten().tolist() == c["gold"], c["name"]


SHAPES = [(256, 256, 128), (256, 1024, 1024), (512, 768, 384), (300, 260, 144),
          (1, 4, 16), (16, 512, 2048), (128, 256, 4096), (257, 516, 272), (64, 100, 80),
          (33, 7, 50)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("trans_b", [False, True])
def test_int8_accumulators_bit_exact(ops, m, n, k, trans_b):
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    want = orc.quant_dot(a, b, orc.I8)
    tb = dev(np.ascontiguousarray(b.T)).t() if trans_b else dev(b)
    got = ops.quant_dot(dev(a), tb).cpu().numpy()
    assert got.dtype == np.int32
    assert np.array_equal(got, want)


# few output tiles and a long K: the split-K form of the kernel (shares of K added into C with
# integer atomics) must still be bit-exact, for any split remainder and for rows past M
SKINNY = [(16, 8192, 8192), (128, 2048, 4096), (1, 256, 2048), (37, 512, 1088), (300, 260, 1024),
          (1024, 1024, 1024), (16, 768, 576)]


@pytest.mark.parametrize("m,n,k", SKINNY)
@pytest.mark.parametrize("trans_b", [False, True])
def test_int8_skinny_split_k_bit_exact(ops, m, n, k, trans_b):
    rng = np.random.default_rng(m + n * 5 + k * 11)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    want = orc.quant_dot(a, b, orc.I8)
    tb = dev(np.ascontiguousarray(b.T)).t() if trans_b else dev(b)
    print("skinny", m, n, k, trans_b, flush=True)
    out = torch.full((m, n + 4), 7, dtype=torch.int32, device="cuda")
    # a second call into the same buffer must not accumulate on top of the first
    for _ in range(2):
        ops.quant_dot(dev(a), tb, out=out[:, :n])
    assert np.array_equal(out[:, :n].cpu().numpy(), want)
    assert (out[:, n:] == 7).all()


def test_int8_skinny_batched(ops):
    rng = np.random.default_rng(5)
    bt, m, n, k = 3, 24, 256, 1536
    a = rng.integers(-128, 128, (bt, m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (bt, k, n), dtype=np.int8)
    want = orc.quant_dot(a, b, orc.I8)
    got = ops.quant_dot(dev(a), dev(b)).cpu().numpy()
    assert np.array_equal(got, want)


def test_int8_extremes_and_batch(ops):
    a = np.full((2, 256, 512), -128, np.int8)
    b = np.full((2, 512, 256), -128, np.int8)
    a[1] = 127
    got = ops.quant_dot(dev(a), dev(b)).cpu().numpy()
    assert np.all(got[0] == 128 * 128 * 512) and np.all(got[1] == -127 * 128 * 512)
    rng = np.random.default_rng(1)
    a = rng.integers(-128, 128, (3, 70, 96), dtype=np.int8)
    b = rng.integers(-128, 128, (3, 96, 52), dtype=np.int8)
    assert np.array_equal(ops.quant_dot(dev(a), dev(b)).cpu().numpy(), orc.quant_dot(a, b, orc.I8))


def test_config1_qdq_matmul_bit_exact(ops):
    """benchmark config 1: X fp32 [256,1024] ~N(0,1) -> quantizelinear(1/32, 0) ->
    quant_dot with W int8 U[-127,127] -> per-channel dequantizelinear, seed 0."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((256, 1024)).astype(np.float32)
    w = rng.integers(-127, 128, (1024, 1024), dtype=np.int8)
    sw = rng.uniform(0.001, 0.01, 1024).astype(np.float32)
    sx = np.float32(1.0 / 32)
    xq_ref = orc.quantizelinear(x, sx, np.int8(0), orc.F32, orc.I8)
    want = orc.qdq_matmul_int8(xq_ref, w, sx, sw)
    xq = ops.quantizelinear(dev(x), dev(np.float32([sx])), dev(np.int8([0])))
    assert np.array_equal(xq.cpu().numpy(), xq_ref)
    got = ops.quant_dot(xq, dev(w), scale_a=dev(np.float32([sx])), scale_b=dev(sw))
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("zp_a,zp_b", [(5, 0), (0, -3), (7, -9)])
@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_int8_dequant_epilogue_bit_exact(ops, zp_a, zp_b, out):
    """Asymmetric zero points (simplify_qdq.cpp:250-279), large accumulators
    (|acc| > 2^24 so a float product would differ) and the truncating converts."""
    rng = np.random.default_rng(11 + zp_a * 3 + zp_b)
    m, n, k = 192, 320, 2048
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    a[:8] = 127
    b[:, :8] = 127
    sa = np.float32(0.0371)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    ot = {"f32": orc.F32, "f16": orc.F16, "bf16": orc.BF16}[out]
    want = orc.qdq_matmul_int8(a, b, sa, sb, zp_a, zp_b, ot)
    ta, tb = dev(a), dev(b)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    got = ops.quant_dot(ta, tb, scale_a=dev(np.float32([sa])), scale_b=dev(sb), zp_a=zp_a, zp_b=zp_b,
                        colsum_b=ops.colsum_i8(tb) if zp_a else None,
                        rowsum_a=ops.rowsum_i8(ta) if zp_b else None, out_dtype=td)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(half_bits(got), want)


# ---- the four-wave kernel: one-pass int8 products with K >= 3072 --------------------------------
# Bare products reach it when the tiles alone fill half the chip (here through the batch), products
# with the dequantizing epilogue whenever no workspace is given.

@pytest.mark.parametrize("m,n,k,batch,trans_b", [
    (300, 520, 3136, 32, False),      # ragged M and N tiles, an odd number of slabs (49)
    (300, 520, 3136, 32, True),
    (256, 512, 3072, 64, False),      # whole tiles, 48 slabs
    (513, 260, 3200, 24, True),       # three tile rows with one live row in the last
])
def test_four_wave_kernel_bare_bit_exact(ops, m, n, k, batch, trans_b):
    rng = np.random.default_rng(m + 3 * n + 7 * k + batch)
    a = rng.integers(-128, 128, (batch, m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (batch, k, n), dtype=np.int8)
    a[0, :4] = 127
    b[0, :, :4] = -128
    want = np.stack([orc.quant_dot(a[i], b[i], orc.I8) for i in range(batch)])
    tb = dev(np.ascontiguousarray(b.transpose(0, 2, 1))).transpose(1, 2) if trans_b else dev(b)
    print("w4 bare", m, n, k, batch, trans_b, flush=True)
    got = ops.quant_dot(dev(a), tb).cpu().numpy()
    assert got.dtype == np.int32 and np.array_equal(got, want)


# The steady state of the four-wave kernels runs in trips of twelve slabs while kt + 17 < K / 64; what
# is left goes through the two-slab loops.  K / 64 = 53 ends the trips at slab 36, 54 at 48; 59 and
# 60 (odd / even with one more trip's worth missing), 65 (a trip boundary plus the longest tail) and
# a K that is not a multiple of 128 (the last A step is half a step).
@pytest.mark.parametrize("k", [3392, 3456, 3776, 3840, 4160, 7744])
@pytest.mark.parametrize("trans_b", [False, True])
def test_four_wave_kernels_trip_boundaries_bit_exact(ops, k, trans_b):
    m, n, batch = 300, 520, 22   # 132 tiles: at least half the chip, so no K split (see above)
    rng = np.random.default_rng(k + trans_b)
    a = rng.integers(-128, 128, (batch, m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (batch, k, n), dtype=np.int8)
    want = np.stack([orc.quant_dot(a[i], b[i], orc.I8) for i in range(batch)])
    tb = dev(np.ascontiguousarray(b.transpose(0, 2, 1))).transpose(1, 2) if trans_b else dev(b)
    print("w4 trips int8", k, trans_b, flush=True)
    got = ops.quant_dot(dev(a), tb).cpu().numpy()
    assert np.array_equal(got, want)
    # fp8 on small integers: every partial sum is exact, so the result is the reference's bit for bit
    a8 = orc.fp8_from_f32(rng.integers(-8, 9, (2, m, k)).astype(np.float32))
    b8 = orc.fp8_from_f32(rng.integers(-8, 9, (2, k, n)).astype(np.float32))
    want8 = np.stack([orc.quant_dot(a8[i], b8[i], orc.FP8) for i in range(2)])
    tb8 = dev(np.ascontiguousarray(b8.transpose(0, 2, 1))).transpose(1, 2) if trans_b else dev(b8)
    print("w4 trips fp8", k, trans_b, flush=True)
    got8 = ops.quant_dot(dev(a8), tb8, fp8=True).cpu().numpy()
    assert np.array_equal(got8, want8)


@pytest.mark.parametrize("m,n,k,trans_b", [(260, 264, 3072, False), (512, 520, 3136, True), (100, 1028, 4160, False)])
@pytest.mark.parametrize("zp_a,zp_b", [(0, 0), (7, -9)])
@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_four_wave_kernel_dequantizing_epilogue_bit_exact(ops, m, n, k, trans_b, zp_a, zp_b, out):
    """Per-row and per-column scales, both zero points, a bias and the truncating converts in the
    epilogue of the four-wave kernel; accumulators beyond 2^24."""
    rng = np.random.default_rng(m + n + k + zp_a)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (n, k) if trans_b else (k, n), dtype=np.int8)
    bm = np.ascontiguousarray(b.T) if trans_b else b
    a[:8] = 127
    bm[:, :8] = 127
    b = np.ascontiguousarray(bm.T) if trans_b else bm
    sa = np.float32(0.0371)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = (rng.standard_normal(n) * 3).astype(np.float32)
    want = orc.qdq_matmul_int8(a, bm, sa, sb, zp_a, zp_b, orc.F32) + bias[None, :]
    ta = dev(a)
    tb = dev(b).T if trans_b else dev(b)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    print("w4 dq", m, n, k, trans_b, zp_a, zp_b, out, flush=True)
    got = ops.quant_dot(ta, tb, scale_a=dev(np.float32([sa])), scale_b=dev(sb), zp_a=zp_a, zp_b=zp_b,
                        colsum_b=ops.colsum_i8(tb) if zp_a else None,
                        rowsum_a=ops.rowsum_i8(ta) if zp_b else None, out_dtype=td, bias=dev(bias))
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        ot = orc.F16 if out == "f16" else orc.BF16
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, ot))


@pytest.mark.parametrize("fp8", [False, True])
def test_four_wave_kernel_unaligned_column_arrays(ops, fp8):
    """Per-column scales, column sums and biases normally come four at a time; arrays that start
    off a 16-byte boundary are read one value at a time.  Both must give the same bits."""
    rng = np.random.default_rng(123 + fp8)
    m, n, k = 260, 264, 3072
    if fp8:
        a = orc.fp8_from_f32(rng.integers(-8, 9, (m, k)).astype(np.float32))
        b = orc.fp8_from_f32(rng.integers(-8, 9, (k, n)).astype(np.float32))
    else:
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    sa = dev(np.float32([0.0371]))
    sb = rng.uniform(0.001, 0.01, n + 1).astype(np.float32)
    bias = (rng.standard_normal(n + 1) * 3).astype(np.float32)
    ta, tb = dev(a), dev(b)
    kw = dict(fp8=True) if fp8 else dict(zp_a=5, colsum_b=None)
    outs = []
    for shift in (0, 1):
        sbt = dev(sb)[shift:shift + n] if shift else dev(np.ascontiguousarray(sb[1:]))
        bt = dev(bias)[shift:shift + n] if shift else dev(np.ascontiguousarray(bias[1:]))
        assert (sbt.data_ptr() % 16 == 0) == (shift == 0)
        if not fp8:
            cs = ops.colsum_i8(tb)
            pad = torch.zeros(n + 1, dtype=torch.int32, device="cuda")
            pad[1:] = cs
            kw["colsum_b"] = pad[1:] if shift else cs
        outs.append(ops.quant_dot(ta, tb, scale_a=sa, scale_b=sbt, out_dtype=torch.float32, bias=bt, **kw))
    assert torch.equal(outs[0], outs[1])
    if not fp8:
        want = orc.qdq_matmul_int8(a, b, np.float32(0.0371), sb[1:], 5, 0, orc.F32) + bias[None, 1:]
        assert np.array_equal(outs[0].cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("k", [1024, 3072])
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("out", ["bare", "f32", "bf16"])
def test_results_through_the_lds_copy_into_strided_batched_views(ops, k, fp8, out):
    """The kernels write C from a row-major copy in the LDS, whole rows of a wave's part per store.
    C here is a view with a row pitch beyond N and a batch stride beyond M x pitch, ragged in M and
    N: every element inside must carry the oracle's bits (operands are small integers, so fp8 sums
    are exact too) and everything around the view must stay untouched.  K = 1024 runs on the
    eight-wave kernels, K = 3072 on the four-wave ones."""
    rng = np.random.default_rng(k + 7 * fp8 + len(out))
    bt, m, n, pitch, rows = 2, 300, 264, 280, 310
    if fp8:
        a = orc.fp8_from_f32(rng.integers(-8, 9, (bt, m, k)).astype(np.float32))
        b = orc.fp8_from_f32(rng.integers(-8, 9, (bt, k, n)).astype(np.float32))
    else:
        a = rng.integers(-128, 128, (bt, m, k), dtype=np.int8)
        b = rng.integers(-128, 128, (bt, k, n), dtype=np.int8)
    sa = np.float32(0.0371)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    td = {"bare": torch.float32 if fp8 else torch.int32, "f32": torch.float32, "bf16": torch.bfloat16}[out]
    whole = torch.full((bt, rows, pitch), 7, dtype=td, device="cuda")
    view = whole[:, :m, :n]
    print("lds copy", k, fp8, out, flush=True)
    if out == "bare":
        ops.quant_dot(dev(a), dev(b), fp8=fp8, out=view)
        want = np.stack([orc.quant_dot(a[i], b[i], orc.FP8 if fp8 else orc.I8) for i in range(bt)])
        assert np.array_equal(view.cpu().numpy(), want)
    else:
        ops.quant_dot(dev(a), dev(b), fp8=fp8, scale_a=dev(np.float32([sa])), scale_b=dev(sb), out_dtype=td, out=view)
        ot = orc.F32 if out == "f32" else orc.BF16
        if fp8:
            want = np.stack([orc.qdq_matmul_fp8(a[i], b[i], sa, sb, ot) for i in range(bt)])
        else:
            want = np.stack([orc.qdq_matmul_int8(a[i], b[i], sa, sb, 0, 0, ot) for i in range(bt)])
        got = view.contiguous()
        if out == "f32":
            assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
        else:
            assert np.array_equal(half_bits(got), want)
    # nothing outside the view was written
    outside = whole.clone()
    outside[:, :m, :n] = 7
    assert bool((outside == 7).all())


def test_four_wave_kernel_per_row_scales(ops):
    rng = np.random.default_rng(77)
    m, n, k = 300, 260, 3072
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    sa = rng.uniform(0.01, 0.05, m).astype(np.float32)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    acc = orc.quant_dot(a, b, orc.I8)
    scale = (sa[:, None] * sb[None, :]).astype(np.float32)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.I32, orc.F32)
    got = ops.quant_dot(dev(a), dev(b), scale_a=dev(sa), scale_b=dev(sb))
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_rowsum_colsum(ops):
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, (130, 1000), dtype=np.int8)
    ta = dev(a)
    assert np.array_equal(ops.rowsum_i8(ta).cpu().numpy(), a.astype(np.int32).sum(1))
    assert np.array_equal(ops.colsum_i8(ta).cpu().numpy(), a.astype(np.int32).sum(0))
    assert np.array_equal(ops.colsum_i8(ta.t()).cpu().numpy(), a.astype(np.int32).sum(1))
    assert np.array_equal(ops.rowsum_i8(ta.t()).cpu().numpy(), a.astype(np.int32).sum(0))


def _fp8_codes(rng, shape, sigma):
    x = rng.normal(0, sigma, shape).astype(np.float32)
    return orc.fp8_from_f32(np.clip(x, -448, 448))


def _fp8_bound(a, b):
    """sum_k |a||b| per output: the scale of the fp32 accumulation error."""
    fa = np.abs(orc.fp8_to_f32(a)).astype(np.float64)
    fb = np.abs(orc.fp8_to_f32(b)).astype(np.float64)
    return fa @ fb


# Tolerance of the fp8 path.  The reference's double accumulator holds the
# exact dot product and rounds once.  v_mfma_f32_16x16x128_f8f6f4 adds each
# group of 128 exact products with a fixed-point window of about 20 bits below
# the largest product of the group (measured: errors up to 2^-15.5 of sum|a||b|
# on operands that span the whole e4m3 range, truncating), then accumulates
# groups in fp32.  An output passes when it is within 1e-3 relative of the
# reference, or (bf16/half outputs) within 1 ulp of the output type, or --
# where the exact sum cancels far below its terms, so that no fp32
# accumulation in another order than the reference's can hold 1e-3 of the
# result -- within 2^-15.5 of sum|a||b| (times the scale).  The last clause is a
# declared deviation from "1e-3 relative or 1 bf16 ulp"; on the benchmark's own
# operand distribution the measured error stays below 2^-19 of sum|a||b| and
# test_full_size_fp8_config3_against_oracle holds the kernel to 2^-18 there and
# bounds the share of outputs that need the clause at all.
FP8_ABS_FLOOR = 2.0**-15.5
FP8_CONFIG3_FLOOR = 2.0**-18


def _fp8_close(got, want, bound):
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    rel = diff <= 1e-3 * np.abs(want)
    need = ~rel & (bound > 0)
    if need.any():    # what the floor clause was asked to cover (shown with pytest -s)
        print("  fp8: %.2e of outputs outside 1e-3 relative, worst error / sum|a||b| = 2^%.2f"
              % (need.mean(), np.log2((diff[need] / bound[need]).max())), flush=True)
    return rel | (diff <= bound * FP8_ABS_FLOOR)


@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (256, 512, 1024), (512, 384, 4096), (96, 132, 272)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_fp8_accumulators(ops, m, n, k, trans_b):
    rng = np.random.default_rng(m + n + k)
    a = _fp8_codes(rng, (m, k), 1.0 * 100)
    b = _fp8_codes(rng, (k, n), 0.02 * 5000)
    want = orc.quant_dot(a, b, orc.FP8)
    tb = dev(np.ascontiguousarray(b.T)).t() if trans_b else dev(b)
    got = ops.quant_dot(dev(a), tb, fp8=True).cpu().numpy()
    assert got.dtype == np.float32
    ok = _fp8_close(got, want, _fp8_bound(a, b))
    assert ok.all(), (np.abs(got - want).max(), (~ok).sum())
    # the bulk is far tighter than the tolerance
    rel = np.abs(got - want) / np.maximum(np.abs(want), 1e-30)
    print("fp8 rel err median %.2e max %.2e; max |diff|/sum|a||b| %.2e" %
          (np.median(rel), rel.max(), (np.abs(got - want) / _fp8_bound(a, b)).max()))
    assert np.median(rel) < 1e-4


def test_fp8_small_integers_are_exact(ops):
    """Operands that are small integers give sums the fp32 accumulator holds
    exactly, so the result must equal the reference bit for bit."""
    rng = np.random.default_rng(2)
    m, n, k = 256, 256, 512
    a = orc.fp8_from_f32(rng.integers(-8, 9, (m, k)).astype(np.float32))
    b = orc.fp8_from_f32(rng.integers(-8, 9, (k, n)).astype(np.float32))
    want = orc.quant_dot(a, b, orc.FP8)
    got = ops.quant_dot(dev(a), dev(b), fp8=True).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_fp8_dequant_epilogue(ops, out):
    """benchmark config 3 at reduced size: amax-scaled fp8 operands, per-tensor
    scales, fp32 accumulate, truncating bf16 output."""
    rng = np.random.default_rng(3)
    m, n, k = 256, 384, 2048
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    sx = np.float32(np.abs(x).max() / 448)
    sw = np.float32(np.abs(w).max() / 448)
    xq = orc.quantizelinear(x, sx, None, orc.F32, orc.FP8)
    wq = orc.quantizelinear(w, sw, None, orc.F32, orc.FP8)
    ot = orc.F32 if out == "f32" else orc.BF16
    want = orc.qdq_matmul_fp8(xq, wq, sx, sw, ot)
    td = torch.float32 if out == "f32" else torch.bfloat16
    got = ops.quant_dot(dev(xq), dev(wq), fp8=True, scale_a=dev(np.float32([sx])),
                        scale_b=dev(np.float32([sw])), out_dtype=td)
    bound = _fp8_bound(xq, wq) * float(sx) * float(sw)
    if out == "f32":
        ok = _fp8_close(got.cpu().numpy(), want, bound)
    else:
        gb = bf16_bits(got)
        gf = orc.bf16_to_f32(gb)
        wf = orc.bf16_to_f32(want)
        ok = (ulp_distance_16(gb, want) <= 1) | _fp8_close(gf, wf, bound)
        # most outputs are identical to the reference's bits
        assert (gb == want).mean() > 0.98
    assert ok.all(), (~ok).sum()


@pytest.mark.parametrize("m,n", [(200, 264), (77, 512), (256, 260), (130, 1000)])
@pytest.mark.parametrize("out", ["f16", "bf16"])
def test_fp8_16bit_outputs_ragged_shapes(ops, m, n, out):
    """16-bit outputs leave the kernel as 16-byte stores built from two lanes' halves when
    N % 8 == 0 (first, second and fourth shape) and as 8-byte or single stores otherwise; rows
    past M and column groups past N are dropped in pairs.  Per-column scales, so a swapped
    half would show."""
    rng = np.random.default_rng(m + n)
    k = 320
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    xq = orc.quantizelinear(x, np.float32(np.abs(x).max() / 448), None, orc.F32, orc.FP8)
    wq = orc.quantizelinear(w, np.float32(np.abs(w).max() / 448), None, orc.F32, orc.FP8)
    sx = np.float32(0.03)
    sw = rng.uniform(0.001, 0.01, n).astype(np.float32)
    ot = orc.F16 if out == "f16" else orc.BF16
    want = orc.qdq_matmul_fp8(xq, wq, sx, sw, ot)
    td = torch.float16 if out == "f16" else torch.bfloat16
    print("fp8 16-bit out", m, n, out, flush=True)
    got = ops.quant_dot(dev(xq), dev(wq), fp8=True, scale_a=dev(np.float32([sx])), scale_b=dev(sw),
                        out_dtype=td)
    gb = got.view(torch.int16).cpu().numpy().view(np.uint16)
    to_f32 = orc.half_to_f32 if out == "f16" else orc.bf16_to_f32
    bound = _fp8_bound(xq, wq) * float(sx) * sw[None, :]
    ok = (ulp_distance_16(gb, want) <= 1) | _fp8_close(to_f32(gb), to_f32(want), bound)
    assert ok.all(), (~ok).sum()
    # most outputs are bit-identical (half keeps three more bits of the fp32 sum than bf16, so fewer
    # of them); a misplaced half would be off by the ratio of two column scales
    assert (gb == want).mean() > (0.97 if out == "bf16" else 0.8)


@pytest.mark.parametrize("m,n,k,trans_b", [(192, 320, 2048, False), (512, 768, 768, True), (100, 260, 128, False),
                                           (33, 50, 40, False), (64, 130, 256, True), (300, 1002, 512, False)])
@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_int8_bias_epilogue_bit_exact(ops, m, n, k, trans_b, out):
    """quant_dot -> dequantizelinear -> add(bias) [-> convert] in one launch: the bias is one more
    fp32 addition (op/binary.hpp:60-90 through add), rounded on its own.  The shapes cover the
    three int8 kernels (N % 4 == 0 large, small, and the any-stride one)."""
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (n, k) if trans_b else (k, n), dtype=np.int8)
    bm = b.T if trans_b else b
    sa = np.float32(0.0371)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = (rng.standard_normal(n) * 3).astype(np.float32)
    bias[:4] = [0.0, -0.0, 1e-30, -1e4]
    zp_a = 3 if m % 2 else 0
    want = orc.qdq_matmul_int8(a, np.ascontiguousarray(bm), sa, sb, zp_a, 0, orc.F32) + bias[None, :]
    assert want.dtype == np.float32
    tb = dev(b).T if trans_b else dev(b)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    print("int8 bias", m, n, k, trans_b, out, flush=True)
    got = ops.quant_dot(dev(a), tb, scale_a=dev(np.float32([sa])), scale_b=dev(sb), zp_a=zp_a,
                        colsum_b=ops.colsum_i8(tb) if zp_a else None, out_dtype=td, bias=dev(bias))
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        ot = orc.F16 if out == "f16" else orc.BF16
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, ot))


@pytest.mark.parametrize("k", [768, 3072])
@pytest.mark.parametrize("out,with_bias", [("f32", True), ("bf16", True), ("f32", False)])
def test_int8_layers_over_shared_activations_in_one_launch(ops, k, out, with_bias):
    """Three layers that read the same activations (the q / k / v projections of an attention block) as one batched
    launch: A with a batch stride of 0, the weights stacked, one vector of column scales and one bias per batch entry
    (MI355_QP_PER_COL_BATCH).  Each batch entry equals the oracle's layer bit for bit, on the eight-wave (K = 768) and
    the four-wave (K = 3072) kernel."""
    m, n, nb = 640, 768, 3
    rng = np.random.default_rng(k + len(out))
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (nb, k, n), dtype=np.int8)
    sa = np.float32(0.0371)
    sb = rng.uniform(0.001, 0.01, (nb, n)).astype(np.float32)
    bias = (rng.standard_normal((nb, n)) * 3).astype(np.float32)
    td = {"f32": torch.float32, "bf16": torch.bfloat16}[out]
    da = dev(a)
    print("int8 shared activations", k, out, with_bias, flush=True)
    got = ops.quant_dot(da.unsqueeze(0).expand(nb, m, k), dev(b), scale_a=dev(np.float32([sa])), scale_b=dev(sb),
                        out_dtype=td, bias=dev(bias) if with_bias else None)
    assert got.shape == (nb, m, n)
    for i in range(nb):
        want = orc.qdq_matmul_int8(a, b[i], sa, sb[i], 0, 0, orc.F32)
        if with_bias:
            want = want + bias[i][None, :]
        if out == "f32":
            assert np.array_equal(got[i].cpu().numpy().view(np.uint32), want.view(np.uint32)), i
        else:
            assert np.array_equal(half_bits(got[i]), orc.convert(want, orc.F32, orc.BF16)), i


def test_column_scales_per_batch_entry_where_no_kernel_has_them(ops):
    """fp8 operands, a bare result and N % 4 != 0 have no kernel with per-batch column scales: refused, not computed
    with the first entry's scales."""
    from amdmigraphx_amd import Mi355Error
    nb, m, k = 2, 64, 256
    sa = dev(np.float32([0.1]))
    for n, fp8 in ((128, True), (130, False)):
        dt = torch.uint8 if fp8 else torch.int8
        a = torch.zeros((nb, m, k), dtype=dt, device="cuda")
        b = torch.zeros((nb, k, n), dtype=dt, device="cuda")
        sb = torch.ones((nb, n), dtype=torch.float32, device="cuda")
        with pytest.raises(Mi355Error):
            ops.quant_dot(a, b, scale_a=sa, scale_b=sb, fp8=fp8)


@pytest.mark.parametrize("m,n,k", [(256, 384, 2048), (200, 264, 320), (77, 130, 192)])
@pytest.mark.parametrize("out", ["f32", "bf16"])
def test_fp8_bias_epilogue(ops, m, n, k, out):
    """The fp8 kernels add the bias to exactly the value they would have stored without one (no
    fused multiply-add): biased output == convert(unbiased fp32 output + bias) bit for bit."""
    rng = np.random.default_rng(m * 3 + n)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    sx = np.float32(np.abs(x).max() / 448)
    sw = np.float32(np.abs(w).max() / 448)
    xq = orc.quantizelinear(x, sx, None, orc.F32, orc.FP8)
    wq = orc.quantizelinear(w, sw, None, orc.F32, orc.FP8)
    bias = (rng.standard_normal(n) * 0.5).astype(np.float32)
    bias[:2] = [0.0, -0.0]
    dsx, dsw = dev(np.float32([sx])), dev(np.float32([sw]))
    print("fp8 bias", m, n, k, out, flush=True)
    plain = ops.quant_dot(dev(xq), dev(wq), fp8=True, scale_a=dsx, scale_b=dsw, out_dtype=torch.float32)
    want = plain.cpu().numpy() + bias[None, :]
    td = torch.float32 if out == "f32" else torch.bfloat16
    got = ops.quant_dot(dev(xq), dev(wq), fp8=True, scale_a=dsx, scale_b=dsw, out_dtype=td, bias=dev(bias))
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        assert np.array_equal(bf16_bits(got), orc.convert(want, orc.F32, orc.BF16))
    # and the unbiased value is the oracle's within the fp8 accumulation bound
    ref = orc.qdq_matmul_fp8(xq, wq, sx, sw, orc.F32)
    assert _fp8_close(plain.cpu().numpy(), ref, _fp8_bound(xq, wq) * float(sx) * float(sw)).all()


@pytest.mark.parametrize("m,n,k,batch,trans_b", [
    (260, 264, 3072, 1, False), (512, 520, 3200, 1, True), (100, 1028, 4224, 1, False),
    (256, 256, 3072, 2, True), (1024, 768, 3968, 1, False)])
def test_fp8_four_wave_kernel_small_integers_exact(ops, m, n, k, batch, trans_b):
    """From K = 3072 on fp8 runs on four waves of 128 x 128 (K a whole number of 128-wide slabs or
    not, an odd and an even number of them, ragged M and N, batches).  Small-integer operands make
    every partial sum exact in fp32, so each element must equal the reference bit for bit whatever
    the order of accumulation: a misplaced fragment, slab or tile shows."""
    rng = np.random.default_rng(m + 3 * n + 7 * k + batch)
    a = orc.fp8_from_f32(rng.integers(-8, 9, (batch, m, k)).astype(np.float32))
    b = orc.fp8_from_f32(rng.integers(-8, 9, (batch, k, n)).astype(np.float32))
    want = np.stack([orc.quant_dot(a[i], b[i], orc.FP8) for i in range(batch)])
    tb = dev(np.ascontiguousarray(b.transpose(0, 2, 1))).transpose(1, 2) if trans_b else dev(b)
    print("fp8 w4 exact", m, n, k, batch, trans_b, flush=True)
    got = ops.quant_dot(dev(a), tb, fp8=True).cpu().numpy()
    assert got.dtype == np.float32 and np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k,trans_b", [(384, 512, 4096, False), (200, 264, 3072, True)])
def test_fp8_four_wave_kernel_accumulators(ops, m, n, k, trans_b):
    """Operands over the whole e4m3 range: the tolerance of the fp8 path, as for the shorter K."""
    rng = np.random.default_rng(m + n + k)
    a = _fp8_codes(rng, (m, k), 1.0 * 100)
    b = _fp8_codes(rng, (k, n), 0.02 * 5000)
    want = orc.quant_dot(a, b, orc.FP8)
    tb = dev(np.ascontiguousarray(b.T)).t() if trans_b else dev(b)
    print("fp8 w4 acc", m, n, k, trans_b, flush=True)
    got = ops.quant_dot(dev(a), tb, fp8=True).cpu().numpy()
    ok = _fp8_close(got, want, _fp8_bound(a, b))
    assert ok.all(), (np.abs(got - want).max(), (~ok).sum())
    rel = np.abs(got - want) / np.maximum(np.abs(want), 1e-30)
    assert np.median(rel) < 1e-4


@pytest.mark.parametrize("m,n,k,trans_b", [(260, 264, 3072, False), (512, 520, 3200, True), (100, 1028, 4224, False),
                                           (77, 130, 3072, False)])
@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("row_scales", [False, True])
def test_fp8_four_wave_kernel_dequantizing_epilogue(ops, m, n, k, trans_b, out, row_scales):
    """Scales per column and per tensor or per row, a bias and the truncating converts in the
    four-wave kernel's epilogue, with 16-byte, 8-byte and single stores (N % 8 == 0, N % 4 == 0,
    neither).  Small-integer operands: the accumulators are exact, so the output must be the
    reference's dequantizelinear -> add -> convert bit for bit."""
    rng = np.random.default_rng(m + n + k)
    a = orc.fp8_from_f32(rng.integers(-8, 9, (m, k)).astype(np.float32))
    bm = orc.fp8_from_f32(rng.integers(-8, 9, (k, n)).astype(np.float32))
    sa = rng.uniform(0.01, 0.05, m).astype(np.float32) if row_scales else np.float32([0.0371])
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = (rng.standard_normal(n) * 3).astype(np.float32)
    acc = orc.quant_dot(a, bm, orc.FP8)
    scale = (sa.reshape(-1, 1) * sb[None, :]).astype(np.float32) * np.ones((m, 1), np.float32)
    want = orc.dequantizelinear(acc, np.ascontiguousarray(scale), None, orc.F32, orc.F32) + bias[None, :]
    assert want.dtype == np.float32
    tb = dev(np.ascontiguousarray(bm.T)).t() if trans_b else dev(bm)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    print("fp8 w4 dq", m, n, k, trans_b, out, row_scales, flush=True)
    got = ops.quant_dot(dev(a), tb, fp8=True, scale_a=dev(sa), scale_b=dev(sb), out_dtype=td, bias=dev(bias))
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        ot = orc.F16 if out == "f16" else orc.BF16
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, ot))


def test_bias_needs_the_epilogue(ops):
    a = dev(np.ones((16, 16), np.int8))
    with pytest.raises(Exception):
        ops.quant_dot(a, a, bias=dev(np.zeros(16, np.float32)))


def _sweep_case(seed):
    rng = np.random.default_rng(1000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    m = int(pick([1, 3, 16, 17, 64, 100, 255, 256, 257, 300]))
    n = int(pick([1, 4, 7, 16, 60, 64, 128, 200, 256, 260]))
    k = int(pick([1, 5, 16, 48, 64, 80, 128, 192, 256, 320, 400]))
    return dict(m=m, n=n, k=k, trans_a=bool(rng.integers(0, 2)), trans_b=bool(rng.integers(0, 2)),
                batch=int(pick([1, 1, 2, 3])), dequant=bool(rng.integers(0, 4) > 0),
                sa_row=bool(rng.integers(0, 2)), sb_col=bool(rng.integers(0, 2)),
                zp_a=int(pick([0, 0, 4, -9])), zp_b=int(pick([0, 0, -3, 11])),
                bias=bool(rng.integers(0, 2)), out=pick(["f32", "f32", "f16", "bf16"]), rng=rng)


@pytest.mark.parametrize("seed", range(48))
def test_int8_seeded_sweep_over_every_dispatch_path(ops, seed):
    """Shapes on and around the tile sizes, transposed views of either operand, batches, every
    epilogue mode: whichever of the three int8 kernels the dispatcher picks, the result is the
    oracle's bit for bit."""
    c = _sweep_case(seed)
    rng, m, n, k, nb = c["rng"], c["m"], c["n"], c["k"], c["batch"]
    a = rng.integers(-128, 128, (nb, m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (nb, k, n), dtype=np.int8)
    da = dev(np.ascontiguousarray(a.transpose(0, 2, 1))).transpose(1, 2) if c["trans_a"] else dev(a)
    db = dev(np.ascontiguousarray(b.transpose(0, 2, 1))).transpose(1, 2) if c["trans_b"] else dev(b)
    if nb == 1:
        da, db = da[0], db[0]
    print("sweep", seed, {x: c[x] for x in c if x != "rng"}, flush=True)
    if not c["dequant"]:
        got = ops.quant_dot(da, db).cpu().numpy().reshape(nb, m, n)
        for i in range(nb):
            assert np.array_equal(got[i], orc.quant_dot(a[i], b[i], orc.I8))
        return
    zp_a, zp_b = (c["zp_a"], c["zp_b"]) if nb == 1 else (0, 0)
    sa = rng.uniform(0.01, 0.05, m if c["sa_row"] else 1).astype(np.float32)
    sb = rng.uniform(0.001, 0.01, n if c["sb_col"] else 1).astype(np.float32)
    bias = (rng.standard_normal(n) * 2).astype(np.float32) if c["bias"] else None
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[c["out"]]
    got = ops.quant_dot(da, db, scale_a=dev(sa), scale_b=dev(sb), zp_a=zp_a, zp_b=zp_b,
                        colsum_b=ops.colsum_i8(db) if zp_a else None,
                        rowsum_a=ops.rowsum_i8(da) if zp_b else None, out_dtype=td,
                        bias=None if bias is None else dev(bias))
    got = got.reshape(nb, m, n)
    for i in range(nb):
        want = orc.qdq_matmul_int8(a[i], b[i], sa.reshape(-1, 1) if c["sa_row"] else sa[0],
                                   sb if c["sb_col"] else sb[0], zp_a, zp_b, orc.F32)
        if bias is not None:
            want = want + bias[None, :]
        if c["out"] == "f32":
            assert np.array_equal(got[i].cpu().numpy().view(np.uint32), want.view(np.uint32))
        else:
            ot = orc.F16 if c["out"] == "f16" else orc.BF16
            assert np.array_equal(half_bits(got[i]), orc.convert(want, orc.F32, ot))


@pytest.mark.parametrize("seed", range(20))
def test_fp8_seeded_sweep_over_every_dispatch_path(ops, seed):
    """The same sweep for fp8 e4m3fn operands (amax-quantized normal data): the float result stays
    within the tolerance of the fp8 matrix instructions whichever kernel runs, with and without the
    scaling epilogue."""
    c = _sweep_case(100 + seed)
    rng, m, n, k = c["rng"], c["m"], c["n"], c["k"]
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    xq = orc.quantizelinear(x, np.float32(max(np.abs(x).max(), 1e-3) / 448), None, orc.F32, orc.FP8)
    wq = orc.quantizelinear(w, np.float32(max(np.abs(w).max(), 1e-3) / 448), None, orc.F32, orc.FP8)
    da = dev(np.ascontiguousarray(xq.T)).t() if c["trans_a"] else dev(xq)
    db = dev(np.ascontiguousarray(wq.T)).t() if c["trans_b"] else dev(wq)
    print("fp8 sweep", seed, {x_: c[x_] for x_ in c if x_ != "rng"}, flush=True)
    bound = _fp8_bound(xq, wq)
    if not c["dequant"]:
        got = ops.quant_dot(da, db, fp8=True).cpu().numpy()
        assert _fp8_close(got, orc.quant_dot(xq, wq, orc.FP8), bound).all()
        return
    sa = np.float32(0.013)
    sb = rng.uniform(0.001, 0.01, n if c["sb_col"] else 1).astype(np.float32)
    want = orc.qdq_matmul_fp8(xq, wq, sa, sb if c["sb_col"] else sb[0], orc.F32)
    got = ops.quant_dot(da, db, fp8=True, scale_a=dev(np.float32([sa])), scale_b=dev(sb),
                        out_dtype=torch.float32).cpu().numpy()
    assert _fp8_close(got, want, bound * float(sa) * (sb[None, :] if c["sb_col"] else float(sb[0]))).all()


@pytest.mark.parametrize("m,n,k", [(5, 7, 3), (64, 48, 300), (130, 257, 96)])
def test_uint8_quant_dot_bare(ops, m, n, k):
    """uint8 x uint8 -> int32 (op/quant_dot.hpp:62-64): exact, also for a transposed B view and
    in batches; with an epilogue the library refuses instead of guessing."""
    from amdmigraphx_amd import Mi355Error
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(0, 256, (2, k, n), dtype=np.uint8)
    want = np.matmul(a.astype(np.int64), b.astype(np.int64))
    assert np.array_equal(orc.quant_dot(a[0], b[0], orc.U8), want[0])
    got = ops.quant_dot(dev(a), dev(b))
    assert got.dtype == torch.int32 and np.array_equal(got.cpu().numpy(), want)
    bt = dev(np.ascontiguousarray(b[0].T)).t()
    assert np.array_equal(ops.quant_dot(dev(a[0]), bt).cpu().numpy(), want[0])
    with pytest.raises(Mi355Error):
        ops.quant_dot(dev(a[0]), dev(b[0]), scale_a=dev(np.float32([0.1])), scale_b=dev(np.float32([0.2])))


def test_argument_errors(ops):
    from amdmigraphx_amd import Mi355Error
    a = torch.zeros((4, 8), dtype=torch.int8, device="cuda")
    b = torch.zeros((9, 4), dtype=torch.int8, device="cuda")
    with pytest.raises(Mi355Error):
        ops.quant_dot(a, b)                       # inner dimensions differ
    with pytest.raises(Mi355Error):
        ops.quant_dot(a, torch.zeros((8, 4), dtype=torch.uint8, device="cuda"))
    out = ops.quant_dot(torch.zeros((0, 8), dtype=torch.int8, device="cuda"),
                        torch.zeros((8, 4), dtype=torch.int8, device="cuda"))
    assert out.shape == (0, 4)


@pytest.mark.parametrize("m,n,k,workspace", [(8192, 8192, 8192, False), (4096, 4096, 4096, False),
                                             (1024, 1024, 1024, False), (1024, 1024, 1024, True),
                                             (128, 8192, 8192, False), (128, 8192, 8192, True),
                                             (16, 8192, 8192, False), (16, 8192, 8192, True)])
def test_full_size_int8_properties(ops, m, n, k, workspace):
    """benchmark config 2 at its real sizes (the square sweep and the skinny shapes), the bare
    call and the call with a split-K workspace: sampled rows against the oracle and row / column
    checksum identities over the whole result."""
    torch.manual_seed(m + k)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
    b = torch.randint(-128, 128, (k, n), dtype=torch.int8, device="cuda")
    print("int8 full size", m, n, k, workspace, flush=True)
    if workspace:
        nbytes = ops.quant_dot_workspace_size(m, n, k)
        if m <= 128:
            assert nbytes > 0, "the skinny shapes are meant to take the split"
        ws = torch.full((max(nbytes, 16),), 0x5A, dtype=torch.uint8, device="cuda")
        c = ops.quant_dot(a, b, workspace=ws)
    else:
        c = ops.quant_dot(a, b)
    rows = sorted({r for r in (0, 1, 15, 16, 127, 255, 256, m // 2 - 1, m // 2, m - 2, m - 1) if 0 <= r < m})
    want = orc.quant_dot(a[rows].cpu().numpy(), b.cpu().numpy(), orc.I8)
    assert np.array_equal(c[rows].cpu().numpy(), want)
    # sum_n C[m, n] == sum_k A[m, k] * (sum_n B[k, n]); all values < 2^53
    lhs = c.double().sum(1)
    rhs = a.double() @ b.double().sum(1)
    assert torch.equal(lhs, rhs)
    # column checksum as well
    lhs = c.double().sum(0)
    rhs = a.double().sum(0) @ b.double()
    assert torch.equal(lhs, rhs)


@pytest.mark.parametrize("n,k", [(768, 768), (3072, 768), (768, 3072)])
def test_full_size_config5_linear_layers(ops, n, k):
    """The quantized MatMuls of benchmark config 5 at their real size -- 32 x 384 = 12288 tokens
    against hidden 768 / FFN 3072, per-tensor activation scale, per-output-channel weight scales,
    bias, fp32 result -- as the one fused launch the lowering makes of them: sampled rows against
    the oracle bit for bit (simplify_qdq.cpp:225-289, dequantizelinear.hpp:60-83, then the add), the
    bare int32 accumulators of the same rows, and a checksum identity over the whole bare result."""
    m = 12288
    torch.manual_seed(n * 3 + k)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
    b = torch.randint(-127, 128, (k, n), dtype=torch.int8, device="cuda")
    rng = np.random.default_rng(n + k)
    sa = np.float32(0.0317)
    sb = rng.uniform(0.0005, 0.002, n).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.02).astype(np.float32)
    print("config 5 linear layer", m, n, k, flush=True)
    got = ops.quant_dot(a, b, scale_a=dev(np.float32([sa])), scale_b=dev(sb), bias=dev(bias),
                        out_dtype=torch.float32)
    bare = ops.quant_dot(a, b)
    rows = [0, 1, 63, 64, 255, 256, 383, 384, 6143, 6144, 12031, 12287]
    ah, bh = a[rows].cpu().numpy(), b.cpu().numpy()
    assert np.array_equal(bare[rows].cpu().numpy(), orc.quant_dot(ah, bh, orc.I8))
    want = orc.qdq_matmul_int8(ah, bh, sa, sb, 0, 0, orc.F32) + bias[None, :]
    assert want.dtype == np.float32
    assert np.array_equal(got[rows].cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert torch.equal(bare.double().sum(1), a.double() @ b.double().sum(1))
    assert torch.equal(bare.double().sum(0), a.double().sum(0) @ b.double())
    # every row of the fused result is the dequantized bare row plus the bias, over the whole result
    scale = torch.from_numpy(np.float32(sa) * sb).cuda()
    whole = (bare.double() * scale.double()[None, :]).float() + dev(bias)[None, :]
    assert torch.equal(got, whole)


def test_graph_replay_of_split_k_and_int4_kernels(ops):
    """A captured HIP graph holding the split-K quant_dot (zero-fill kernel + integer
    atomics) and the int4 GEMM must give the eager result on every replay, with eager
    work and synchronisation between the replays."""
    rng = np.random.default_rng(21)
    m, n, k = 16, 1024, 4096
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    want = orc.quant_dot(a, b, orc.I8)
    ta, tb = dev(a), dev(b)
    out = torch.empty((m, n), dtype=torch.int32, device="cuda")
    ops.quant_dot(ta, tb, out=out)  # warm up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.quant_dot(ta, tb, out=out)
    for rep in range(3):
        out.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want), rep
        # eager work between the replays
        assert np.array_equal(ops.quant_dot(ta, tb).cpu().numpy(), want)


@pytest.mark.parametrize("k,n", [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)])
def test_full_size_fp8_config3_shapes(ops, k, n):
    """benchmark config 3 at its real sizes (M = 4096).  fp8 codes that hold small integers
    make every partial sum an integer below 2^24, which the fp32 accumulator and the MFMA's
    internal alignment hold exactly: the fp8 quant_dot must then equal the int8 quant_dot of
    the same integers, element for element, over the whole result.  The bf16 epilogue is
    checked against the float result with the scale applied (one truncation)."""
    m = 4096
    g = torch.Generator(device="cuda")
    g.manual_seed(k + n)
    ai = torch.randint(-4, 5, (m, k), dtype=torch.int8, device="cuda", generator=g)
    bi = torch.randint(-4, 5, (k, n), dtype=torch.int8, device="cuda", generator=g)
    # e4m3 codes of the integers -4..4
    lut = torch.tensor([int(orc.fp8_from_f32(np.float32([v]))[0]) for v in range(-4, 5)],
                       dtype=torch.uint8, device="cuda")
    a8 = lut[(ai.long() + 4)]
    b8 = lut[(bi.long() + 4)]
    print("fp8 full size", k, n, flush=True)
    want = ops.quant_dot(ai, bi)                    # int32, exact
    got = ops.quant_dot(a8, b8, fp8=True)           # float
    assert torch.equal(got, want.float())
    s1 = torch.tensor([0.0078125], device="cuda")    # powers of two: the scaled value is exact
    s2 = torch.tensor([0.25], device="cuda")
    out = ops.quant_dot(a8, b8, fp8=True, scale_a=s1, scale_b=s2, out_dtype=torch.bfloat16)
    exact = want.float() * (0.0078125 * 0.25)
    # bf16 by truncation: never above the exact value in magnitude, within one bf16 step
    diff = (exact.abs() - out.float().abs())
    assert (diff >= 0).all()
    assert (diff <= exact.abs() * 2.0**-7).all()
    assert (out.float().sign() * exact.sign() >= 0).all()


def _config3_operands(k, n, m=4096):
    """benchmark config 3: bf16 activations ~N(0,1) and weights ~N(0,0.02), each quantized to fp8
    e4m3fn with its per-tensor scale amax / 448 (generated and quantized on the device; the
    quantizelinear kernel has its own parity tests)."""
    from amdmigraphx_amd import ops
    g = torch.Generator(device="cuda")
    g.manual_seed(k * 7 + n)
    x = torch.randn((m, k), device="cuda", generator=g).bfloat16().float()
    w = (torch.randn((k, n), device="cuda", generator=g) * 0.02).bfloat16().float()
    sx = (x.abs().max() / 448).reshape(1)
    sw = (w.abs().max() / 448).reshape(1)
    xq = ops.quantizelinear(x, sx, None, out_type=ops.DT.FP8)
    wq = ops.quantizelinear(w, sw, None, out_type=ops.DT.FP8)
    return xq, wq, sx, sw


@pytest.mark.parametrize("k,n", [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)])
def test_full_size_fp8_config3_against_oracle(ops, k, n):
    """benchmark config 3 at its real sizes and on its own distribution: sampled rows of the bf16
    result against the oracle (exact sum, one rounding, scale, truncation to bf16), with the
    tolerance accounted for clause by clause.  The contract is 1e-3 relative or 1 bf16 ulp; the
    third clause (a floor relative to sum|a||b|, for sums that cancel) is a declared deviation and
    the test bounds how many outputs need it."""
    m = 4096
    xq, wq, sx, sw = _config3_operands(k, n, m)
    print("fp8 config 3 vs oracle", k, n, flush=True)
    out = ops.quant_dot(xq, wq, fp8=True, scale_a=sx, scale_b=sw, out_dtype=torch.bfloat16)
    acc = ops.quant_dot(xq, wq, fp8=True)
    rows = [0, 1, 31, 32, 255, 256, 2047, 2048, 4094, 4095]
    a = xq[rows].cpu().numpy()
    b = wq.cpu().numpy()
    s1 = np.float32(sx.cpu().numpy()[0])
    s2 = np.float32(sw.cpu().numpy()[0])
    want_acc = orc.quant_dot(a, b, orc.FP8)
    want = orc.qdq_matmul_fp8(a, b, s1, s2, orc.BF16)
    bound = _fp8_bound(a, b)
    # fp32 accumulators
    got_acc = acc[rows].cpu().numpy()
    diff = np.abs(got_acc.astype(np.float64) - want_acc.astype(np.float64))
    rel_ok = diff <= 1e-3 * np.abs(want_acc)
    ulp_ok = diff <= np.abs(want_acc) * 2.0**-8          # one bf16 step of the value, at least
    floor_ok = diff <= bound * FP8_CONFIG3_FLOOR
    assert (rel_ok | ulp_ok | floor_ok).all()
    frac_rel = 1.0 - rel_ok.mean()
    frac_floor = (~(rel_ok | ulp_ok)).mean()
    print("  fp32: outside 1e-3 relative: %.2e of outputs; need the floor: %.2e; worst error / sum|a||b| = 2^%.2f"
          % (frac_rel, frac_floor, np.log2((diff / bound).max())), flush=True)
    assert frac_rel < 2e-2
    assert frac_floor < 5e-3
    # bf16 outputs
    gb = bf16_bits(out[rows])
    gf = orc.bf16_to_f32(gb).astype(np.float64)
    wf = orc.bf16_to_f32(want).astype(np.float64)
    d16 = np.abs(gf - wf)
    one_ulp = ulp_distance_16(gb, want) <= 1
    rel16 = d16 <= 1e-3 * np.abs(wf)
    floor16 = d16 <= bound * FP8_CONFIG3_FLOOR * float(s1) * float(s2)
    assert (one_ulp | rel16 | floor16).all()
    frac16 = (~(one_ulp | rel16)).mean()
    print("  bf16: identical bits %.4f; within 1 ulp %.6f; need the floor: %.2e"
          % ((gb == want).mean(), one_ulp.mean(), frac16), flush=True)
    assert (gb == want).mean() > 0.98
    assert frac16 < 3e-3


# skinny bare int8 products with a workspace: K is split over workgroups that write partial tiles,
# a second kernel adds them; the result must be the bits of the one-pass product (int32 sums are
# exact in any order) and of the oracle
@pytest.mark.parametrize("m,n,k,batch,trans_b", [
    (16, 1024, 4096, 1, False), (16, 1024, 4096, 1, True), (128, 512, 2048, 1, False), (1, 256, 8192, 1, True),
    (33, 260, 1024, 2, True), (40, 300, 1600, 1, True), (8, 256, 2112, 1, False),
    (16, 1023, 4096, 1, True), (40, 301, 1600, 2, True),  # N % 4 != 0: padded partial rows, scalar stores
    # benchmark config 2, the skinny shapes at full size
    (16, 8192, 8192, 1, False), (128, 8192, 8192, 1, True), (128, 8192, 8192, 1, False),
])
def test_int8_split_k_with_workspace_bit_exact(ops, m, n, k, batch, trans_b):
    g = torch.Generator().manual_seed(m * 7 + n + k)
    a = torch.randint(-128, 128, (batch, m, k), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (batch, n, k) if trans_b else (batch, k, n), dtype=torch.int8, generator=g)
    da, db = a.cuda(), b.cuda()
    dbv = db.transpose(1, 2) if trans_b else db
    bytes_ = ops.quant_dot_workspace_size(m, n, k, batch, trans_b)
    assert bytes_ > 0, "these shapes are meant to take the split"
    assert bytes_ % (batch * m * ((n + 3) // 4 * 4) * 4) == 0  # partial rows are padded to 4 columns
    ws = torch.full((bytes_ // 4,), 0x55555555, dtype=torch.int32, device="cuda")
    got = ops.quant_dot(da, dbv, workspace=ws)
    ref = ops.quant_dot(da, dbv)
    assert torch.equal(got, ref)
    want = torch.matmul(a.double(), (b.transpose(1, 2) if trans_b else b).double()).to(torch.int32)
    assert torch.equal(got.cpu(), want)
    # a workspace that is too small is not an error: the call takes the path without one
    small = torch.empty(64, dtype=torch.int32, device="cuda")
    assert torch.equal(ops.quant_dot(da, dbv, workspace=small), ref)
    # second call with the same workspace (stale partial sums from the first), into a view of a
    # wider buffer: the columns beside it stay as they were
    wide = torch.full((batch, m, n + 8), 7, dtype=torch.int32, device="cuda")
    ops.quant_dot(da, dbv, workspace=ws, out=wide[:, :, :n])
    assert torch.equal(wide[:, :, :n], ref)
    assert (wide[:, :, n:] == 7).all()


def test_workspace_size_is_zero_where_no_split_pays(ops):
    assert ops.quant_dot_workspace_size(8192, 8192, 8192) == 0
    assert ops.quant_dot_workspace_size(16, 64, 128) == 0


@pytest.mark.parametrize("m,n,k,trans_b", [(16, 1024, 4096, False), (128, 768, 3072, True), (40, 304, 1600, False),
                                           (1, 512, 8192, True), (8, 256, 2112, False), (24, 250, 2048, True),
                                           (17, 49, 4608, True),
                                           # benchmark config 2, the skinny shapes at full size
                                           (16, 8192, 8192, False), (128, 8192, 8192, True)])
@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
def test_int8_split_k_with_workspace_dequantizing_epilogue(ops, m, n, k, trans_b, out):
    """The skinny fused linear layer: the second kernel of the workspace split applies the
    dequantizelinear epilogue (scales per row and per column, both zero points, bias, convert) to
    the summed partial tiles.  Required: the bits of the oracle, which are also those of the
    one-pass kernel."""
    rng = np.random.default_rng(m * 13 + n + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (n, k) if trans_b else (k, n), dtype=np.int8)
    bm = np.ascontiguousarray(b.T) if trans_b else b
    sa = rng.uniform(0.01, 0.05, m).astype(np.float32)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = (rng.standard_normal(n) * 3).astype(np.float32)
    bias[:2] = [0.0, -0.0]
    zp_a, zp_b = (3, -2) if m % 16 else (0, 0)
    # (an int8 product whose N is no multiple of 4 takes a bias on another kernel: none there)
    use_bias = n % 4 == 0
    want = orc.qdq_matmul_int8(a, bm, sa[:, None], sb[None, :], zp_a, zp_b, orc.F32)
    if use_bias:
        want = want + bias[None, :]
    assert want.dtype == np.float32
    tb = dev(b).T if trans_b else dev(b)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    nbytes = ops.quant_dot_workspace_size(m, n, k, 1, trans_b)
    assert nbytes > 0
    ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device="cuda")
    print("int8 workspace dq", m, n, k, trans_b, out, flush=True)
    kw = dict(scale_a=dev(sa), scale_b=dev(sb), zp_a=zp_a, zp_b=zp_b,
              colsum_b=ops.colsum_i8(tb) if zp_a else None, rowsum_a=ops.rowsum_i8(dev(a)) if zp_b else None,
              out_dtype=td, bias=dev(bias) if use_bias else None)
    got = ops.quant_dot(dev(a), tb, workspace=ws, **kw)
    one_pass = ops.quant_dot(dev(a), tb, **kw)
    assert torch.equal(got.view(torch.int32 if out == "f32" else torch.int16),
                       one_pass.view(torch.int32 if out == "f32" else torch.int16))
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        ot = orc.F16 if out == "f16" else orc.BF16
        assert np.array_equal(half_bits(got), orc.convert(want, orc.F32, ot))


@pytest.mark.parametrize("m,n,k,trans_b", [(16, 1024, 4096, False), (128, 768, 3072, True), (40, 304, 1600, False),
                                           (1, 512, 8192, True), (64, 256, 2112, False)])
@pytest.mark.parametrize("out", ["bare", "f32", "bf16"])
def test_fp8_split_k_with_workspace(ops, m, n, k, trans_b, out):
    """fp8 skinny shapes with a workspace: K is cut into equal slices (float partial sums, added in
    a fixed order by the second kernel, which also applies scale, bias and convert).  The sums are
    floats in another order than the one-pass kernel's, so the requirement is the fp8 tolerance
    against the oracle (as for the one-pass kernel) and the same bits on every call."""
    rng = np.random.default_rng(m + 3 * n + k)
    a = _fp8_codes(rng, (m, k), 100.0)
    b = _fp8_codes(rng, (k, n), 100.0)
    tb = dev(np.ascontiguousarray(b.T)).t() if trans_b else dev(b)
    nbytes = ops.quant_dot_workspace_size(m, n, k, 1, trans_b, fp8=True)
    assert nbytes > 0 and nbytes % (m * n * 4) == 0 and (k // 64) % (nbytes // (m * n * 4)) == 0
    ws = torch.full((nbytes,), 0x7F, dtype=torch.uint8, device="cuda")  # NaN patterns if read unwritten
    print("fp8 workspace", m, n, k, trans_b, out, flush=True)
    if out == "bare":
        want = orc.quant_dot(a, b, orc.FP8)
        got = ops.quant_dot(dev(a), tb, fp8=True, workspace=ws)
        again = ops.quant_dot(dev(a), tb, fp8=True, workspace=ws)
        assert torch.equal(got.view(torch.int32), again.view(torch.int32))
        assert _fp8_close(got.cpu().numpy(), want, _fp8_bound(a, b)).all()
        rel = np.abs(got.cpu().numpy() - want) / np.maximum(np.abs(want), 1e-30)
        assert np.median(rel) < 1e-4
        return
    sx, sw = np.float32(0.0123), np.float32(0.00371)
    sb = (rng.uniform(0.5, 1.5, n) * sw).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.5).astype(np.float32)
    td = torch.float32 if out == "f32" else torch.bfloat16
    kw = dict(fp8=True, scale_a=dev(np.float32([sx])), scale_b=dev(sb), out_dtype=td, bias=dev(bias))
    got = ops.quant_dot(dev(a), tb, workspace=ws, **kw)
    again = ops.quant_dot(dev(a), tb, workspace=ws, **kw)
    assert torch.equal(got.view(torch.int32 if out == "f32" else torch.int16),
                       again.view(torch.int32 if out == "f32" else torch.int16))
    # the epilogue on top of this path's own bare sums, bit for bit: fp32 scale product, one
    # multiply, one add, convert
    bare = ops.quant_dot(dev(a), tb, fp8=True, workspace=ws).cpu().numpy()
    step = (bare * (sx * sb)[None, :]).astype(np.float32) + bias[None, :]
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), step.view(np.uint32))
    else:
        assert np.array_equal(bf16_bits(got), orc.convert(step, orc.F32, orc.BF16))
    # and the oracle's value within the fp8 tolerance
    ref = orc.quant_dot(a, b, orc.FP8).astype(np.float64) * (np.float64(sx) * sb.astype(np.float64))[None, :] + bias
    bound = _fp8_bound(a, b) * float(sx) * sb.astype(np.float64)[None, :]
    gf = got.float().cpu().numpy()
    if out == "f32":
        assert _fp8_close(gf, ref, bound).all()
    else:
        assert ((np.abs(gf - ref) <= np.abs(ref) * 2.0**-7) | _fp8_close(gf, ref, bound)).all()
