"""GPU parity of quant_dot over a constant B reordered ahead of time (mi355_quant_dot_prepack +
mi355_quant_dot_prepacked) against the CPU oracle and against mi355_quant_dot_bias."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev, bf16_bits, half_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k", [(16, 64), (48, 192), (256, 1024), (512, 8192), (8192, 512), (1040, 832)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_int8_accumulators_are_exact(ops, m, n, k, trans_b):
    """every split of K over the waves (1 .. 16 waves per tile column, remainders), both source
    layouts of B, rows short of 16"""
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    tb = dev(np.ascontiguousarray(b.T)).t() if trans_b else dev(b)
    print("prepacked int8", m, n, k, trans_b, flush=True)
    pk = ops.quant_dot_prepack(tb)
    assert pk is not None and pk.numel() == n * k
    got = ops.quant_dot_prepacked(dev(a), pk, n).cpu().numpy()
    want = a.astype(np.int64) @ b.astype(np.int64)
    assert got.dtype == np.int32 and np.array_equal(got, want)


@pytest.mark.parametrize("out", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("zp", [(0, 0), (3, 0), (0, -5), (7, -2)])
def test_int8_dequantizing_epilogue_matches_the_one_pass_kernel_and_the_oracle(ops, out, zp):
    rng = np.random.default_rng(11)
    m, n, k = 13, 320, 1280
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    sa = rng.uniform(0.01, 0.05, m).astype(np.float32)
    sb = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[out]
    colsum = dev(b.astype(np.int32).sum(0).astype(np.int32))
    rowsum = dev(a.astype(np.int32).sum(1).astype(np.int32))
    kw = dict(scale_a=dev(sa), scale_b=dev(sb), zp_a=zp[0], zp_b=zp[1], colsum_b=colsum, rowsum_a=rowsum,
              out_dtype=td, bias=dev(bias))
    pk = ops.quant_dot_prepack(dev(b))
    got = ops.quant_dot_prepacked(dev(a), pk, n, **kw)
    other = ops.quant_dot(dev(a), dev(b), **kw)
    assert torch.equal(got.view(torch.int16) if out != "f32" else got.view(torch.int32),
                       other.view(torch.int16) if out != "f32" else other.view(torch.int32))
    ot = {"f32": orc.F32, "f16": orc.F16, "bf16": orc.BF16}[out]
    deq = orc.qdq_matmul_int8(a, b, sa[:, None], sb[None, :], zp[0], zp[1])
    want = (deq + bias[None, :]).astype(np.float32)
    if out == "f32":
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        gb = half_bits(got) if out == "f16" else bf16_bits(got)
        assert np.array_equal(gb, orc.convert(want, orc.F32, ot))


@pytest.mark.parametrize("fmt", [True, "e5m2"])
@pytest.mark.parametrize("m,n,k", [(16, 256, 2048), (3, 64, 320), (16, 1024, 8192)])
def test_fp8_within_tolerance_and_exact_on_small_integers(ops, fmt, m, n, k):
    rng = np.random.default_rng(k + m)
    enc, dec, ot = (orc.fp8_from_f32, orc.fp8_to_f32, orc.FP8) if fmt is True else \
        (orc.bf8_from_f32, orc.bf8_to_f32, orc.BF8)
    a = enc(rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.5)
    b = enc(rng.integers(-8, 9, (k, n)).astype(np.float32))
    pk = ops.quant_dot_prepack(dev(b), fp8=fmt)
    got = ops.quant_dot_prepacked(dev(a), pk, n, fp8=fmt).cpu().numpy()
    assert np.array_equal(got, orc.quant_dot(a, b, ot))
    a = enc(np.clip(rng.normal(0, 30, (m, k)), -400, 400).astype(np.float32))
    b = enc(np.clip(rng.normal(0, 2, (k, n)), -400, 400).astype(np.float32))
    pk = ops.quant_dot_prepack(dev(b), fp8=fmt)
    sa, sb = np.float32([0.02]), rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    got = ops.quant_dot_prepacked(dev(a), pk, n, fp8=fmt, scale_a=dev(sa), scale_b=dev(sb), bias=dev(bias),
                                  out_dtype=torch.float32).cpu().numpy()
    want = (orc.qdq_matmul_fp8(a, b, sa, sb, orc.F32, fp8_type=ot) + bias[None, :]).astype(np.float32)
    bound = (np.abs(dec(a)).astype(np.float64) @ np.abs(dec(b)).astype(np.float64)) * 0.02 * sb[None, :]
    diff = np.abs(got.astype(np.float64) - want)
    ok = (diff <= 1e-3 * np.abs(want)) | (diff <= bound * 2.0**-15.5)
    assert ok.all(), (~ok).sum()


def test_full_size_config2_rows(ops):
    """M = 16, N = K = 8192 (benchmark config 2): every accumulator against an int64 product on
    the device's own copy, the fused layer against the one-pass kernel."""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    a = torch.randint(-128, 128, (16, 8192), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-128, 128, (8192, 8192), dtype=torch.int8, device="cuda", generator=g)
    pk = ops.quant_dot_prepack(b)
    got = ops.quant_dot_prepacked(a, pk, 8192)
    want = ops.quant_dot(a, b)
    assert torch.equal(got, want)
    rows = a[[0, 15]].cpu().numpy().astype(np.int64) @ b.cpu().numpy().astype(np.int64)
    assert np.array_equal(got[[0, 15]].cpu().numpy(), rows)


def test_declines_other_shapes(ops):
    from amdmigraphx_amd import Mi355Error
    assert ops.quant_dot_prepack(torch.zeros((64, 24), dtype=torch.int8, device="cuda")) is None   # N % 16
    assert ops.quant_dot_prepack(torch.zeros((96, 32), dtype=torch.int8, device="cuda")) is None   # K % 64
    pk = ops.quant_dot_prepack(torch.zeros((64, 32), dtype=torch.int8, device="cuda"))
    with pytest.raises(Mi355Error):                                                                # 17 rows
        ops.quant_dot_prepacked(torch.zeros((17, 64), dtype=torch.int8, device="cuda"), pk, 32)
