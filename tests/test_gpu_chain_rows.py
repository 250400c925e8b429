"""GPU test of mi355_chain_rows_f32 through the C ABI: the chain machine with the row-mean step.  A layer
normalisation written as its separate operators (reduce_mean, sub, mul, reduce_mean, add, rsqrt, mul, mul, add:
the expansion of ONNX LayerNormalization) must come out of the one kernel with the bits the CPU oracle gives for
the operators one after another (op/reduce_mean.hpp:34-50 and the binary / unary operators)."""
import ctypes

import numpy as np
import pytest
import torch

from amdmigraphx_amd import capi
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

LOAD, BINARY, UNARY, SAVE, ROW_MEAN = 0, 1, 2, 3, 4
ADD, SUB, MUL, DIV = 0, 1, 2, 3
SQRT, RSQRT = 1, 2
SAVED, SELF = -1, -2


class Step(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("op", ctypes.c_int32), ("src", ctypes.c_int32),
                ("reversed", ctypes.c_int32)]


def run_rows(steps, inputs, strides, rows, cols, entry="mi355_chain_rows_f32"):
    arr = (Step * len(steps))(*[Step(*s) for s in steps])
    ptrs = (ctypes.c_void_p * len(inputs))(*[t.data_ptr() for t in inputs])
    sr = (ctypes.c_int64 * len(inputs))(*[s[0] for s in strides])
    sc = (ctypes.c_int32 * len(inputs))(*[s[1] for s in strides])
    out = torch.full((rows, cols), float("nan"), dtype=torch.float32, device="cuda")
    st = getattr(capi.lib(), entry)(ctypes.cast(arr, ctypes.c_void_p), len(steps), ptrs, sr, sc, len(inputs),
                                    ctypes.c_void_p(out.data_ptr()), rows, cols,
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return st, out


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# inputs: 0 a, 1 b, 2 eps (one value), 3 gamma [cols], 4 beta [cols]
CORE = [(SAVE, 0, 0, 0), (ROW_MEAN, 0, 0, 0),
        (BINARY, SUB, SAVED, 1),           # x - mean
        (SAVE, 0, 0, 0), (BINARY, MUL, SELF, 0), (ROW_MEAN, 0, 0, 0)]
FORMS = {
    # x = a + b, rsqrt and a product, scale and shift: the library has a kernel of its own for this step list
    "sum_rsqrt_affine": [(LOAD, 0, 0, 0), (BINARY, ADD, 1, 0)] + CORE +
                        [(BINARY, ADD, 2, 0), (UNARY, RSQRT, 0, 0), (BINARY, MUL, SAVED, 1),
                         (BINARY, MUL, 3, 0), (BINARY, ADD, 4, 0)],
    # x = a, sqrt and a quotient, nothing behind: likewise
    "plain_sqrt": [(LOAD, 0, 0, 0)] + CORE +
                  [(BINARY, ADD, 2, 0), (UNARY, SQRT, 0, 0), (BINARY, DIV, SAVED, 1)],
    # the operands of three steps the other way round: the general step machine
    "machine": [(LOAD, 0, 0, 0), (BINARY, ADD, 1, 1)] + CORE +
               [(BINARY, ADD, 2, 1), (UNARY, RSQRT, 0, 0), (BINARY, MUL, SAVED, 0),
                (BINARY, MUL, 3, 0), (BINARY, ADD, 4, 0), (BINARY, SUB, 1, 1)],
}


def layer_norm_by_operators(form, a, b, eps, g, beta):
    x = a if form == "plain_sqrt" else orc.binary_f32("add", a, b)
    mean = orc.reduce_mean_f32(x, [-1])
    xc = orc.binary_f32("sub", x, mean)
    var = orc.reduce_mean_f32(orc.binary_f32("mul", xc, xc), [-1])
    ve = orc.binary_f32("add", var, np.float32(eps))
    if form == "plain_sqrt":
        return orc.binary_f32("div", xc, orc.unary_f32("sqrt", ve))
    y = orc.binary_f32("mul", xc, orc.unary_f32("rsqrt", ve))
    y = orc.binary_f32("add", orc.binary_f32("mul", y, g), beta)
    return orc.binary_f32("sub", b, y) if form == "machine" else y


# every register count of the kernels (4, 12, 16, 32, 64 columns per lane), ragged rows and row counts
@pytest.mark.parametrize("form", sorted(FORMS))
@pytest.mark.parametrize("rows,cols", [(1, 1), (5, 7), (33, 200), (7, 256), (130, 257), (1027, 768), (64, 1000),
                                       (9, 1024), (6, 1500), (5, 2048), (3, 3001), (2, 4096)])
def test_layer_norm_in_one_kernel_equals_its_operators(form, rows, cols):
    rng = np.random.default_rng(rows * 10007 + cols)
    a = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    b = rng.standard_normal((rows, cols)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    beta = rng.standard_normal(cols).astype(np.float32)
    eps = np.float32(1e-5)
    want = layer_norm_by_operators(form, a, b, eps, g, beta)
    d = [torch.from_numpy(t).cuda() for t in (a, b, np.array([eps], np.float32), g, beta)]
    print("chain rows", form, rows, cols, flush=True)
    st, out = run_rows(FORMS[form], d, [(cols, 1), (cols, 1), (0, 0), (0, 1), (0, 1)], rows, cols)
    assert st == 0
    assert np.array_equal(bits(out.cpu().numpy()), bits(want))


def test_the_two_kernels_agree_on_special_values():
    """Rows with infinities, NaNs and zeros, a constant row (variance 0) and a row of denormals: the kernel for the
    recognised step list and the step machine (the same list with the commutative eps sum written the other way
    round) give the same bits."""
    rows, cols = 8, 300
    rng = np.random.default_rng(11)
    a = rng.standard_normal((rows, cols)).astype(np.float32)
    a[1, 5] = np.inf
    a[2, 7] = np.nan
    a[3, :] = 2.5
    a[4, :] = 0.0
    a[5, :] = np.float32(1e-41) * rng.integers(1, 100, cols).astype(np.float32)
    a[6, 0] = -np.inf
    a[6, 1] = np.inf
    b = rng.standard_normal((rows, cols)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    beta = rng.standard_normal(cols).astype(np.float32)
    d = [torch.from_numpy(t).cuda() for t in (a, b, np.array([1e-5], np.float32), g, beta)]
    strides = [(cols, 1), (cols, 1), (0, 0), (0, 1), (0, 1)]
    fast = FORMS["sum_rsqrt_affine"]
    slow = [(BINARY, ADD, 2, 1) if s == (BINARY, ADD, 2, 0) else s for s in fast]
    assert slow != fast
    st1, out1 = run_rows(fast, d, strides, rows, cols)
    st2, out2 = run_rows(slow, d, strides, rows, cols)
    assert st1 == 0 and st2 == 0
    o1, o2 = out1.cpu().numpy(), out2.cpu().numpy()
    finite = np.isfinite(o1)
    assert np.array_equal(finite, np.isfinite(o2)) and np.array_equal(np.isnan(o1), np.isnan(o2))
    assert np.array_equal(bits(o1[finite]), bits(o2[finite]))
    assert np.isfinite(o1[0]).all() and np.isfinite(o1[3]).all() and np.isnan(o1[2]).all()


def test_row_mean_alone_is_reduce_mean_and_broadcast():
    rows, cols = 1000, 768
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((rows, cols)) * 100).astype(np.float32)
    dx = torch.from_numpy(x).cuda()
    st, out = run_rows([(LOAD, 0, 0, 0), (ROW_MEAN, 0, 0, 0)], [dx], [(cols, 1)], rows, cols)
    assert st == 0
    mean = torch.empty(rows, dtype=torch.float32, device="cuda")
    assert capi.lib().mi355_reduce_mean_f32(ctypes.c_void_p(dx.data_ptr()), ctypes.c_void_p(mean.data_ptr()), rows, cols,
                                            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int32), mean[:, None].expand(rows, cols).contiguous().view(torch.int32))
    assert np.array_equal(bits(mean.cpu().numpy()), bits(orc.reduce_mean_f32(x, [-1]).reshape(rows)))


def test_strided_rows_and_a_value_per_row():
    """An input that is a slice of wider rows (row stride above cols) and one that holds one value per row."""
    rows, cols, pitch = 37, 300, 512
    rng = np.random.default_rng(4)
    wide = rng.standard_normal((rows, pitch)).astype(np.float32)
    per_row = rng.standard_normal(rows).astype(np.float32)
    d = [torch.from_numpy(wide).cuda(), torch.from_numpy(per_row).cuda()]
    st, out = run_rows([(LOAD, 0, 0, 0), (BINARY, MUL, 1, 0), (SAVE, 0, 0, 0), (ROW_MEAN, 0, 0, 0), (BINARY, SUB, SAVED, 0)],
                       d, [(pitch, 1), (1, 0)], rows, cols)
    assert st == 0
    v = orc.binary_f32("mul", wide[:, :cols], per_row[:, None])
    want = orc.binary_f32("sub", orc.reduce_mean_f32(v, [-1]), v)
    assert np.array_equal(bits(out.cpu().numpy()), bits(want))


def test_bad_arguments_are_rejected():
    x = torch.zeros(4, 8, device="cuda")
    ok = [(LOAD, 0, 0, 0), (ROW_MEAN, 0, 0, 0)]
    assert run_rows(ok, [x], [(8, 1)], 4, 8)[0] == 0
    assert run_rows(ok, [x], [(8, 1)], 4, 8, entry="mi355_chain_f32")[0] != 0   # the elementwise machine has no rows
    assert run_rows([(ROW_MEAN, 0, 0, 0)], [x], [(8, 1)], 4, 8)[0] != 0          # no LOAD first
    assert run_rows(ok, [x], [(8, 2)], 4, 8)[0] != 0                            # column stride 2
    assert run_rows([(LOAD, 0, 0, 0), (5, 0, 0, 0)], [x], [(8, 1)], 4, 8)[0] != 0
    wide = torch.zeros(1, 4100, device="cuda")
    assert run_rows(ok, [wide], [(4100, 1)], 1, 4100)[0] != 0                    # more columns than a wave holds
    assert run_rows(ok, [x], [(8, 1)], 0, 8)[0] == 0                             # empty: nothing to do
