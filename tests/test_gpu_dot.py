"""Float `dot` on the device against the CPU oracle (gemm_naive: double accumulation, one rounding):
the default entry point bit for bit, the fp32 matrix-core entry point within fp32 accumulation
error -- K * 2^-24 of sum|a||b| -- which is far inside the 1e-3 relative the path's float outputs
are held to."""
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


@pytest.mark.parametrize("bt,m,n,k,trans_b", [(1, 64, 64, 64, False), (12, 384, 384, 64, True), (12, 384, 64, 384, False),
                                              (3, 100, 36, 52, False), (2, 33, 130, 260, True)])
def test_float_dot_exact_and_fp32_accumulating(ops, bt, m, n, k, trans_b):
    rng = np.random.default_rng(bt + m + n + k)
    a = rng.standard_normal((bt, m, k)).astype(np.float32)
    b = rng.standard_normal((bt, n, k) if trans_b else (bt, k, n)).astype(np.float32)
    bv = np.swapaxes(b, 1, 2) if trans_b else b
    want = orc.dot(a, bv, orc.F32)
    tb = dev(b).transpose(1, 2) if trans_b else dev(b)
    got = ops.dot(dev(a), tb).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    fast = ops.dot(dev(a), tb, fp32acc=True).cpu().numpy()
    mag = np.abs(a).astype(np.float64) @ np.abs(bv).astype(np.float64)
    err = np.abs(fast.astype(np.float64) - want.astype(np.float64))
    assert (err <= mag * k * 2.0**-24).all(), (err / mag).max()
    # with the scale of attention scores: float(sum) * scale, one more fp32 rounding
    s = torch.tensor([0.125], device="cuda")
    assert np.array_equal(ops.dot(dev(a), tb, scale=s).cpu().numpy(), want * np.float32(0.125))
    scaled = ops.dot(dev(a), tb, scale=s, fp32acc=True).cpu().numpy()
    assert (np.abs(scaled.astype(np.float64) - want * 0.125) <= mag * k * 2.0**-27 + 1e-30).all()


@pytest.mark.parametrize("trans_a", [False, True])
@pytest.mark.parametrize("trans_b", [False, True])
def test_float_dot_whole_tiles_every_layout(ops, trans_a, trans_b):
    """Each of the four operand layouts of the 16-byte-load kernel on whole tiles (rows or columns contiguous, for
    either operand), bit for bit."""
    bt, m, n, k = 2, 128, 192, 192
    rng = np.random.default_rng(77 + 2 * trans_a + trans_b)
    a = rng.standard_normal((bt, k, m) if trans_a else (bt, m, k)).astype(np.float32)
    b = rng.standard_normal((bt, n, k) if trans_b else (bt, k, n)).astype(np.float32)
    av = np.swapaxes(a, 1, 2) if trans_a else a
    bv = np.swapaxes(b, 1, 2) if trans_b else b
    want = orc.dot(np.ascontiguousarray(av), np.ascontiguousarray(bv), orc.F32)
    ta = dev(a).transpose(1, 2) if trans_a else dev(a)
    tb = dev(b).transpose(1, 2) if trans_b else dev(b)
    print("float dot whole tiles", trans_a, trans_b, flush=True)
    got = ops.dot(ta, tb).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("k", [80, 96, 112, 128, 400])
@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
def test_float_dot_three_steps_in_flight_every_remainder(ops, k, trans_a, trans_b):
    """Tiles inside the matrices keep three K steps of operands in flight from K = 96 on, in trips of three steps with
    the one or two steps left over at the end; the tiles on the matrix edges (here the last 36 rows and 20 columns)
    and shorter sums take the plain loop.  Every number of left-over steps, every layout, bit for bit."""
    bt, m, n = 2, 128 + 36, 64 + 20
    rng = np.random.default_rng(500 + k + 2 * trans_a + trans_b)
    a = rng.standard_normal((bt, k, m) if trans_a else (bt, m, k)).astype(np.float32)
    b = rng.standard_normal((bt, n, k) if trans_b else (bt, k, n)).astype(np.float32)
    av = np.swapaxes(a, 1, 2) if trans_a else a
    bv = np.swapaxes(b, 1, 2) if trans_b else b
    want = orc.dot(np.ascontiguousarray(av), np.ascontiguousarray(bv), orc.F32)
    ta = dev(a).transpose(1, 2) if trans_a else dev(a)
    tb = dev(b).transpose(1, 2) if trans_b else dev(b)
    print("float dot trips", k, trans_a, trans_b, flush=True)
    got = ops.dot(ta, tb).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    fast = ops.dot(ta, tb, fp32acc=True).cpu().numpy()
    mag = np.abs(av).astype(np.float64) @ np.abs(bv).astype(np.float64)
    assert (np.abs(fast.astype(np.float64) - want) <= mag * k * 2.0**-24 + 1e-30).all()


@pytest.mark.parametrize("b,h,rows,width", [(2, 3, 40, 16), (1, 4, 128, 64), (3, 2, 70, 20)])
def test_float_dot_writes_its_result_head_merged(b, h, rows, width):
    """mi355_dot_batch2_strided: probabilities [b, h, rows, rows] times values seen as [b, h, rows, width] (a view of
    [b, rows, h, width] storage), the result written straight into [b, rows, h, width] memory -- what transpose(0, 2, 1, 3)
    + contiguous of the dense result would give -- bit for bit, and nothing outside it touched."""
    import ctypes
    from amdmigraphx_amd import capi
    rng = np.random.default_rng(b * 100 + rows)
    probs = rng.standard_normal((b, h, rows, rows)).astype(np.float32)
    vals = rng.standard_normal((b, rows, h, width)).astype(np.float32)
    want = orc.dot(probs.reshape(b * h, rows, rows),
                   np.ascontiguousarray(vals.transpose(0, 2, 1, 3)).reshape(b * h, rows, width), orc.F32)
    want = want.reshape(b, h, rows, width).transpose(0, 2, 1, 3)
    dp, dv = dev(probs), dev(vals)
    out = torch.full((b, rows, h, width), float("nan"), dtype=torch.float32, device="cuda")
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    print("float dot head-merged", b, h, rows, width, flush=True)
    st = capi.lib().mi355_dot_batch2_strided(
        vp(dp), vp(dv), vp(out), 3, rows, width, rows,
        rows, 1, h * width, 1,                 # A rows / k strides, B k / n strides
        h * width,                             # ldc
        b, h,
        h * rows * rows, rows * rows,          # A: batch, head
        rows * h * width, width,               # B: batch, head (the view)
        rows * h * width, width,               # C: batch, head
        None, 0, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert st == 0
    assert np.array_equal(out.cpu().numpy().view(np.uint32), np.ascontiguousarray(want).view(np.uint32))


def test_strided_result_bad_arguments_are_rejected():
    import ctypes
    from amdmigraphx_amd import capi
    x = torch.zeros(2 * 2 * 8 * 8, dtype=torch.float32, device="cuda")
    vp = ctypes.c_void_p(x.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call(ldc=8, bo=2, bi=2, sco=128, sci=64):
        return capi.lib().mi355_dot_batch2_strided(vp, vp, vp, 3, 8, 8, 8, 8, 1, 8, 1, ldc, bo, bi,
                                                   128, 64, 128, 64, sco, sci, None, 0, st)
    assert call(ldc=4) != 0                    # rows of C shorter than N
    assert call(sco=-1) != 0 and call(sci=-1) != 0
    assert call(bo=-1) != 0
    assert call(bo=70000, bi=1) != 0           # more batch entries than one launch addresses
    assert call(bo=0) == 0                     # nothing to do
    torch.cuda.synchronize()


def test_fp32_accumulation_is_float32_only(ops):
    from amdmigraphx_amd import Mi355Error
    a = torch.zeros((16, 16), dtype=torch.float16, device="cuda")
    with pytest.raises(Mi355Error):
        ops.dot(a, a, fp32acc=True)
