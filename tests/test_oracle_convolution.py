"""The oracle's convolution against the reference's known answers and against an independent
restatement (explicit zero padding, window slices, numpy integer / double sums)."""
import numpy as np
import pytest

from oracle import oracle as orc


def test_reference_known_answers(golden):
    for c in golden["convolution"]:
        is_int = c["type"] == "int8"
        dt = np.int8 if is_int else np.float32
        nx, nw = int(np.prod(c["x_lens"])), int(np.prod(c["w_lens"]))
        x = np.arange(nx) if c["x"] == "iota" else np.array(c["x"])
        w = np.arange(nw) if c["w"] == "iota" else np.array(c["w"])
        x = x.astype(dt).reshape(c["x_lens"])
        w = w.astype(dt).reshape(c["w_lens"])
        got = orc.convolution(x, w, orc.I8 if is_int else orc.F32, c["padding"], c["stride"], c["dilation"],
                              c["group"])
        if is_int:
            assert got.dtype == np.int32
            assert got.flatten().tolist() == c["gold"], c["name"]
        else:
            np.testing.assert_allclose(got.flatten(), np.float32(c["gold"]), rtol=2e-6, atol=1e-6, err_msg=c["name"])


def brute(x, w, padding, stride, dilation, group):
    """Independent form: pad with zeros, slice the dilated window, sum products in int64."""
    n, c, h, wd = x.shape
    o, cg, kh, kw = w.shape
    ph, pw = padding[0], padding[1]
    ph2, pw2 = (padding[2], padding[3]) if len(padding) == 4 else (ph, pw)
    xp = np.zeros((n, c, h + ph + ph2, wd + pw + pw2), np.int64)
    xp[:, :, ph:ph + h, pw:pw + wd] = x
    oh = orc.conv_out_len(h, kh, ph, stride[0], dilation[0], ph2)
    ow = orc.conv_out_len(wd, kw, pw, stride[1], dilation[1], pw2)
    og = o // group
    out = np.zeros((n, o, oh, ow), np.int64)
    for oc in range(o):
        g = oc // og
        xs = xp[:, g * cg:(g + 1) * cg]
        for y in range(oh):
            for xx in range(ow):
                y0, x0 = y * stride[0], xx * stride[1]
                win = xs[:, :, y0:y0 + dilation[0] * (kh - 1) + 1:dilation[0],
                         x0:x0 + dilation[1] * (kw - 1) + 1:dilation[1]]
                out[:, oc, y, xx] = (win * w[oc].astype(np.int64)[None]).sum(axis=(1, 2, 3))
    return out


@pytest.mark.parametrize("shape,wshape,padding,stride,dilation,group", [
    ((2, 4, 9, 7), (6, 4, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((1, 6, 8, 8), (4, 3, 3, 2), (0, 1), (2, 1), (1, 2), 2),
    ((3, 8, 5, 11), (8, 1, 3, 3), (2, 2), (1, 3), (2, 1), 8),
    ((2, 3, 6, 6), (5, 3, 1, 1), (0, 0), (2, 2), (1, 1), 1),
    ((1, 2, 7, 7), (2, 2, 5, 5), (2, 2), (1, 1), (1, 1), 1),
    ((2, 3, 8, 9), (4, 3, 3, 3), (0, 1, 2, 0), (2, 2), (1, 1), 1),   # low and high padding differ
    ((1, 2, 6, 6), (2, 2, 3, 3), (2, 0, 0, 1), (1, 1), (1, 1), 1),
])
def test_int8_against_brute_force(shape, wshape, padding, stride, dilation, group):
    rng = np.random.default_rng(sum(shape) + sum(wshape))
    x = rng.integers(-128, 128, shape, dtype=np.int8)
    w = rng.integers(-128, 128, wshape, dtype=np.int8)
    got = orc.convolution(x, w, orc.I8, padding, stride, dilation, group)
    want = brute(x, w, padding, stride, dilation, group)
    assert got.shape == want.shape
    assert np.array_equal(got.astype(np.int64), want)


def test_one_by_one_convolution_is_a_matrix_product():
    rng = np.random.default_rng(4)
    x = rng.integers(-128, 128, (2, 16, 5, 6), dtype=np.int8)
    w = rng.integers(-128, 128, (7, 16, 1, 1), dtype=np.int8)
    got = orc.convolution(x, w, orc.I8)
    want = np.einsum("oc,nchw->nohw", w[:, :, 0, 0].astype(np.int64), x.astype(np.int64))
    assert np.array_equal(got.astype(np.int64), want)


def test_fp8_products_are_exact_in_double():
    # fp8 codes as small integers and halves: every product and the sum are exact, so the float
    # result equals the integer arithmetic on the decoded values
    rng = np.random.default_rng(6)
    vals = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, -0.5, -1.0, -2.0, -4.0], np.float32)
    x = rng.choice(vals, (1, 3, 6, 6)).astype(np.float32)
    w = rng.choice(vals, (4, 3, 3, 3)).astype(np.float32)
    xq, wq = orc.fp8_from_f32(x), orc.fp8_from_f32(w)
    got = orc.convolution(xq, wq, orc.FP8, (1, 1))
    want = orc.convolution(x, w, orc.F32, (1, 1))
    assert got.dtype == np.float32
    assert np.array_equal(got, want)


def brute_nd(x, w, padding, stride, dilation, group):
    """Independent form for any number of spatial axes: pad with zeros, slice the dilated window,
    sum products in int64."""
    nd = x.ndim - 2
    lo, hi = list(padding[:nd]), list(padding[nd:] if len(padding) == 2 * nd else padding[:nd])
    xp = np.zeros(x.shape[:2] + tuple(x.shape[2 + i] + lo[i] + hi[i] for i in range(nd)), np.int64)
    xp[(slice(None), slice(None)) + tuple(slice(lo[i], lo[i] + x.shape[2 + i]) for i in range(nd))] = x
    out_sp = [orc.conv_out_len(x.shape[2 + i], w.shape[2 + i], lo[i], stride[i], dilation[i], hi[i]) for i in range(nd)]
    o, cg = w.shape[:2]
    og = o // group
    out = np.zeros((x.shape[0], o, *out_sp), np.int64)
    for oc in range(o):
        g = oc // og
        xs = xp[:, g * cg:(g + 1) * cg]
        for pos in np.ndindex(*out_sp):
            win = xs[(slice(None), slice(None)) + tuple(
                slice(pos[i] * stride[i], pos[i] * stride[i] + dilation[i] * (w.shape[2 + i] - 1) + 1, dilation[i])
                for i in range(nd))]
            out[(slice(None), oc) + pos] = (win * w[oc].astype(np.int64)[None]).sum(axis=tuple(range(1, nd + 2)))
    return out


@pytest.mark.parametrize("shape,wshape,padding,stride,dilation,group", [
    ((2, 4, 5, 6, 7), (6, 4, 3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    ((1, 6, 6, 5, 4), (4, 3, 2, 3, 1), (1, 0, 2), (2, 1, 1), (1, 2, 1), 2),
    ((2, 4, 7, 4, 5), (4, 1, 3, 2, 2), (0, 1, 0, 2, 0, 1), (1, 2, 3), (2, 1, 1), 4),   # low / high padding
    ((1, 3, 4, 4, 4), (2, 3, 1, 1, 1), (0, 0, 0), (2, 2, 2), (1, 1, 1), 1),
    ((3, 2, 9), (4, 2, 3), (1,), (2,), (2,), 1),                                      # one spatial axis
    ((2, 4, 11), (6, 2, 4), (2, 0), (1,), (1,), 2),
])
def test_int8_one_and_three_spatial_axes_against_brute_force(shape, wshape, padding, stride, dilation, group):
    rng = np.random.default_rng(sum(shape) * 7 + sum(wshape))
    x = rng.integers(-128, 128, shape, dtype=np.int8)
    w = rng.integers(-128, 128, wshape, dtype=np.int8)
    got = orc.convolution(x, w, orc.I8, padding, stride, dilation, group)
    want = brute_nd(x, w, padding, stride, dilation, group)
    assert got.shape == want.shape
    assert np.array_equal(got.astype(np.int64), want)


def test_depth_one_volume_is_the_two_dimensional_convolution():
    rng = np.random.default_rng(11)
    x = rng.integers(-128, 128, (2, 4, 6, 7), dtype=np.int8)
    w = rng.integers(-128, 128, (3, 4, 3, 2), dtype=np.int8)
    flat = orc.convolution(x, w, orc.I8, (1, 0), (1, 2), (1, 1))
    vol = orc.convolution(x[:, :, None], w[:, :, None], orc.I8, (0, 1, 0), (1, 1, 2), (1, 1, 1))
    assert np.array_equal(vol[:, :, 0], flat)
