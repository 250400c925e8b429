"""GPU test of mi355_softmax_f32 against the CPU oracle (ref_softmax, src/targets/ref/lowering.cpp:281-312:
e = float(exp(double(x) - max)), the sum of e in double, float(double(e) / sum)).  The device takes the library
exponential and the division only where a cheaper evaluation could round differently, so the results are the
oracle's bits except where the two math libraries' exp differ in the last place of a double next to a float
rounding boundary: at most a handful of elements in millions, one unit in the last place each."""
import ctypes

import numpy as np
import pytest
import torch

from amdmigraphx_amd import capi
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def softmax_on_device(x):
    rows, cols = x.shape
    dx = torch.from_numpy(x).cuda()
    out = torch.empty_like(dx)
    st = capi.lib().mi355_softmax_f32(ctypes.c_void_p(dx.data_ptr()), ctypes.c_void_p(out.data_ptr()), rows, cols,
                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert st == 0
    return out.cpu().numpy()


def units_apart(a, b):
    return np.abs(a.view(np.int32).astype(np.int64) - b.view(np.int32).astype(np.int64))


# rows held in registers (up to 1024 columns) and the general kernel; spreads from attention scores to
# values whose exponentials reach the float denormals and zero
@pytest.mark.parametrize("rows,cols", [(4099, 384), (1000, 128), (333, 1000), (37, 2500), (3, 5), (64, 1)])
@pytest.mark.parametrize("spread", [1.0, 8.0, 40.0])
def test_softmax_matches_the_oracle(rows, cols, spread):
    rng = np.random.default_rng(rows + cols + int(spread))
    x = (rng.standard_normal((rows, cols)) * spread).astype(np.float32)
    want = orc.softmax_f32(x, 1)
    print("softmax", rows, cols, spread, flush=True)
    got = softmax_on_device(x)
    apart = units_apart(got, want)
    assert apart.max() <= 1 and np.count_nonzero(apart) <= 2 + x.size // 1000000, (apart.max(), np.count_nonzero(apart))
    assert np.allclose(got.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)


def test_masked_and_special_rows():
    """Additive masks (-1e9, -inf), rows of one value, huge values, a NaN: the same as the oracle, element for element."""
    cols = 384
    rng = np.random.default_rng(5)
    x = rng.standard_normal((9, cols)).astype(np.float32)
    x[0, 100:] = -1e9
    x[1, 5:] = -np.inf
    x[2, :] = 3.25
    x[3, :] = -3e38
    x[4, 0] = 3e38
    x[5, :] = np.linspace(-120, 0, cols, dtype=np.float32)     # through the denormal exponentials down to zero
    x[6, :] = np.linspace(-90, -80, cols, dtype=np.float32) + 50
    x[7, 17] = np.nan
    want = orc.softmax_f32(x, 1)
    got = softmax_on_device(x)
    ok = ~np.isnan(want)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert units_apart(got[ok], want[ok]).max() <= 1
    assert np.array_equal(got[:5], want[:5])
