"""GPU test of mi355_chain_f32 through the C ABI: a chain of float operators in one kernel must
give, bit for bit, what the same IEEE operations give one after another (numpy float32 here; the
single-operator entry points mi355_binary_f32 / mi355_unary_f32 for the math-library functions)."""
import ctypes

import numpy as np
import pytest
import torch

from amdmigraphx_amd import capi

pytestmark = pytest.mark.gpu

LOAD, BINARY, UNARY, SAVE = 0, 1, 2, 3
ADD, SUB, MUL, DIV = 0, 1, 2, 3
ERF, SQRT, RSQRT, EXP, TANH, NEG = 0, 1, 2, 3, 4, 5
SAVED, SELF = -1, -2


class Step(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("op", ctypes.c_int32), ("src", ctypes.c_int32),
                ("reversed", ctypes.c_int32)]


def run_chain(steps, inputs, strides, rows, cols, out=None):
    """inputs: device tensors; strides: (row stride, column stride) per input"""
    arr = (Step * len(steps))(*[Step(*s) for s in steps])
    ptrs = (ctypes.c_void_p * len(inputs))(*[t.data_ptr() for t in inputs])
    sr = (ctypes.c_int64 * len(inputs))(*[s[0] for s in strides])
    sc = (ctypes.c_int32 * len(inputs))(*[s[1] for s in strides])
    if out is None:
        out = torch.empty(rows, cols, dtype=torch.float32, device="cuda")
    st = capi.lib().mi355_chain_f32(ctypes.cast(arr, ctypes.c_void_p), len(steps), ptrs, sr, sc, len(inputs),
                                    ctypes.c_void_p(out.data_ptr()), rows, cols,
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return st, out


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# the last two shapes have enough rows for the four-rows-per-pass form, with a ragged last group
@pytest.mark.parametrize("rows,cols", [(33, 200), (7, 203), (1, 4), (300, 1024), (5, 1), (9001, 256), (8195, 203)])
def test_exact_operators_match_numpy(rows, cols):
    rng = np.random.default_rng(rows * 1000 + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32) * 3
    y = rng.uniform(0.5, 3.0, (rows, cols)).astype(np.float32)
    bias = rng.standard_normal(cols).astype(np.float32)
    per_row = rng.uniform(0.5, 2.0, rows).astype(np.float32)
    one = np.float32([1.25])
    dx, dy, db, dr, d1 = (torch.from_numpy(a).cuda() for a in (x, y, bias, per_row, one))
    # ((x + bias) / per_row - y) * 1.25, then y - that, then squared, then 1/sqrt(. + y), negated
    steps = [(LOAD, 0, 0, 0), (BINARY, ADD, 2, 0), (BINARY, DIV, 3, 0), (BINARY, SUB, 1, 0),
             (BINARY, MUL, 4, 0), (BINARY, SUB, 1, 1), (BINARY, MUL, SELF, 0), (BINARY, ADD, 1, 0),
             (UNARY, RSQRT, 0, 0), (UNARY, NEG, 0, 0)]
    st, out = run_chain(steps, [dx, dy, db, dr, d1], [(cols, 1), (cols, 1), (0, 1), (1, 0), (0, 0)], rows, cols)
    assert st == 0
    t = (x + bias[None, :]) / per_row[:, None]
    t = (t - y) * one[0]
    t = y - t
    t = t * t
    t = t + y
    t = np.float32(1.0) / np.sqrt(t)
    t = -t
    assert np.array_equal(bits(out.cpu().numpy()), bits(t))


def test_saved_value_and_reversed_division():
    rows, cols = 19, 64
    rng = np.random.default_rng(5)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    y = rng.uniform(0.5, 3.0, (rows, cols)).astype(np.float32)
    dx, dy = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    # saved = x + y; value = sqrt(y + y); result = saved / value, then value - saved order check
    steps = [(LOAD, 0, 0, 0), (BINARY, ADD, 1, 0), (SAVE, 0, 0, 0), (LOAD, 0, 1, 0), (BINARY, ADD, SELF, 0),
             (UNARY, SQRT, 0, 0), (BINARY, DIV, SAVED, 1), (BINARY, SUB, SAVED, 0)]
    st, out = run_chain(steps, [dx, dy], [(cols, 1), (cols, 1)], rows, cols)
    assert st == 0
    saved = x + y
    t = saved / np.sqrt(y + y)
    t = t - saved
    assert np.array_equal(bits(out.cpu().numpy()), bits(t))


def test_math_functions_match_the_single_operator_kernels():
    rows, cols = 40, 256
    rng = np.random.default_rng(9)
    x = rng.standard_normal((rows, cols)).astype(np.float32) * 2
    dx = torch.from_numpy(x).cuda()
    lib = capi.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = dx.clone()
    for op in (ERF, EXP, TANH):
        nxt = torch.empty_like(want)
        assert lib.mi355_unary_f32(op, ctypes.c_void_p(want.data_ptr()), ctypes.c_void_p(nxt.data_ptr()),
                                   want.numel(), stream) == 0
        want = nxt
    torch.cuda.synchronize()
    st, out = run_chain([(LOAD, 0, 0, 0), (UNARY, ERF, 0, 0), (UNARY, EXP, 0, 0), (UNARY, TANH, 0, 0)],
                        [dx], [(cols, 1)], rows, cols)
    assert st == 0
    assert torch.equal(out.view(torch.int32), want.view(torch.int32))
    ref = np.tanh(np.exp(np.vectorize(__import__("math").erf)(x.astype(np.float64))))
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=1e-5, atol=1e-6)


def test_unaligned_views_take_the_scalar_form():
    rows, cols = 9, 200
    rng = np.random.default_rng(11)
    big = rng.standard_normal((rows, cols + 4)).astype(np.float32)
    dbig = torch.from_numpy(big).cuda()
    view = dbig[:, 1:1 + cols]  # starts 4 bytes off a 16-byte boundary
    y = rng.standard_normal((rows, cols)).astype(np.float32)
    dy = torch.from_numpy(y).cuda()
    st, out = run_chain([(LOAD, 0, 0, 0), (BINARY, MUL, 1, 0), (BINARY, ADD, 0, 0)], [view, dy],
                        [(cols + 4, 1), (cols, 1)], rows, cols)
    assert st == 0
    t = big[:, 1:1 + cols] * y
    t = t + big[:, 1:1 + cols]
    assert np.array_equal(bits(out.cpu().numpy()), bits(t))


def test_bad_arguments_are_rejected():
    x = torch.zeros(4, 8, device="cuda")
    ok = [(LOAD, 0, 0, 0), (UNARY, NEG, 0, 0)]
    assert run_chain(ok, [x], [(8, 1)], 4, 8)[0] == 0
    assert run_chain([(UNARY, NEG, 0, 0)], [x], [(8, 1)], 4, 8)[0] != 0           # no LOAD first
    assert run_chain([(LOAD, 0, 1, 0)], [x], [(8, 1)], 4, 8)[0] != 0              # input index out of range
    assert run_chain([(LOAD, 0, 0, 0), (BINARY, 7, 0, 0)], [x], [(8, 1)], 4, 8)[0] != 0
    assert run_chain([(LOAD, 0, 0, 0), (BINARY, ADD, -3, 0)], [x], [(8, 1)], 4, 8)[0] != 0
    assert run_chain([(LOAD, 0, 0, 0), (9, 0, 0, 0)], [x], [(8, 1)], 4, 8)[0] != 0
    assert run_chain(ok, [x], [(8, 2)], 4, 8)[0] != 0                             # column stride 2
    assert run_chain([(LOAD, 0, 0, 0)] + [(UNARY, NEG, 0, 0)] * 24, [x], [(8, 1)], 4, 8)[0] != 0
    assert run_chain(ok, [x], [(8, 1)], 0, 8)[0] == 0                             # empty: nothing to do


@pytest.mark.parametrize("rows,cols", [(33, 200), (7, 203), (1, 4), (300, 1024), (5, 1), (9001, 256), (8195, 203)])
@pytest.mark.parametrize("zero_point", [None, -7])
def test_quantizing_chain_equals_chain_then_quantizelinear(rows, cols, zero_point):
    """mi355_chain_f32_q8 against mi355_chain_f32 followed by mi355_quantizelinear (one scale and one
    zero point for the tensor), byte for byte; values that saturate both ways, ties and a NaN are in."""
    rng = np.random.default_rng(rows * 7 + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32) * 40
    x.flat[0] = 1e9
    x.flat[-1] = -1e9
    if x.size > 8:
        x.flat[3] = np.nan
        x.flat[5] = 0.75     # (0.75 + 0.75) / 0.5 = 3.0; 0.625 -> 2.5: a tie that goes to even
        x.flat[6] = 0.625
    y = np.full((rows, cols), 0.0, np.float32)
    y.flat[5:7] = x.flat[5:7] if x.size > 8 else 0
    scale = np.float32([0.5])
    dx, dy, ds = (torch.from_numpy(a).cuda() for a in (x, y, scale))
    steps = [(LOAD, 0, 0, 0), (BINARY, ADD, 1, 0)]
    arr = (Step * len(steps))(*[Step(*s) for s in steps])
    ptrs = (ctypes.c_void_p * 2)(dx.data_ptr(), dy.data_ptr())
    sr = (ctypes.c_int64 * 2)(cols, cols)
    sc = (ctypes.c_int32 * 2)(1, 1)
    dz = torch.tensor([zero_point], dtype=torch.int8, device="cuda") if zero_point is not None else None
    zp_ptr = ctypes.c_void_p(dz.data_ptr()) if dz is not None else None
    got = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    print("chain q8", rows, cols, zero_point, flush=True)
    st = capi.lib().mi355_chain_f32_q8(ctypes.cast(arr, ctypes.c_void_p), 2, ptrs, sr, sc, 2,
                                       ctypes.c_void_p(ds.data_ptr()), zp_ptr, ctypes.c_void_p(got.data_ptr()),
                                       rows, cols, stream)
    assert st == 0
    st, mid = run_chain(steps, [dx, dy], [(cols, 1), (cols, 1)], rows, cols)
    assert st == 0
    want = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
    st = capi.lib().mi355_quantizelinear(ctypes.c_void_p(mid.data_ptr()), capi.DT.F32, ctypes.c_void_p(ds.data_ptr()),
                                         0, 0, zp_ptr, 0, 0, ctypes.c_void_p(want.data_ptr()), capi.DT.I8, rows, cols,
                                         stream)
    assert st == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    w = want.cpu().numpy()
    assert w.flat[0] == 127 and w.flat[-1] == -128
