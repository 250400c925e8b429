"""The oracle's float operators (softmax, reduce_mean, gather, binary, unary) against the
reference's own known answers and against closed forms."""
import math

import numpy as np

from oracle import oracle as orc


def test_softmax_reference_known_answers(golden):
    """test/ref/softmax.cpp:33-107.  The second case reduces over axis 1 of a
    [5, 3, 4, 2] tensor: a wrong axis stride or a max / sum taken over the wrong
    elements cannot reproduce 120 expected values.  The reference compares with
    its RMS rule; the printed expectations carry 8 digits."""
    assert len(golden["softmax"]) == 2
    for c in golden["softmax"]:
        x = np.float32(c["a"]).reshape(c["shape"]["lens"])
        got = orc.softmax_f32(x, c["axis"]).flatten()
        gold = np.float32(c["gold"])
        assert np.allclose(got, gold, rtol=2e-6, atol=2e-7), c["name"]


def test_softmax_definition():
    rng = np.random.default_rng(0)
    x = rng.normal(0, 3, (7, 33)).astype(np.float32)
    got = orc.softmax_f32(x, -1)
    # step by step as ref_softmax does it
    mx = x.astype(np.float64).max(axis=1, keepdims=True)
    e = np.exp(x.astype(np.float64) - mx).astype(np.float32)
    s = np.zeros(7)
    for j in range(33):
        s += e[:, j].astype(np.float64)
    want = (e.astype(np.float64) / s[:, None]).astype(np.float32)
    assert np.array_equal(got, want)
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-6)
    # shift invariance and the uniform case
    assert np.allclose(orc.softmax_f32(x + 5, -1), got, atol=1e-6)
    assert np.array_equal(orc.softmax_f32(np.zeros((2, 4), np.float32), 1), np.full((2, 4), 0.25, np.float32))


def test_reduce_mean_reference_known_answers(golden):
    """test/ref/reduce_mean.cpp:33-195: exact equality, as the reference's tests demand."""
    assert len(golden["reduce_mean"]) == 4
    for c in golden["reduce_mean"]:
        x = np.float32(c["input"]).reshape(c["shape"]["lens"])
        got = orc.reduce_mean_f32(x, c["axes"])
        assert got.flatten().tolist() == [float(v) for v in c["gold"]], c["name"]
        shp = [1 if d in c["axes"] else n for d, n in enumerate(c["shape"]["lens"])]
        assert list(got.shape) == shp


def test_reduce_mean_accumulates_in_double():
    # 2^24 + 1 is not a float: a float accumulator would lose the ones
    x = np.float32([[16777216.0] + [1.0] * 255])
    got = orc.reduce_mean_f32(x, [-1])
    want = np.float32((16777216.0 + 255.0) / 256.0)
    assert got[0, 0] == want
    rng = np.random.default_rng(1)
    y = rng.normal(0, 1, (5, 1000)).astype(np.float32)
    assert np.array_equal(orc.reduce_mean_f32(y, [1])[:, 0],
                          (np.cumsum(y.astype(np.float64), axis=1)[:, -1] / 1000.0).astype(np.float32))


def test_gather_reference_known_answers(golden):
    """test/ref/gather.cpp:59-214: axes 0, 1 and -1, negative indices, scalar indices."""
    assert len(golden["gather"]) == 7
    for c in golden["gather"]:
        data = (np.arange(c["data_count"], dtype=np.float32) + np.float32(c["data_iota_start"]))
        data = data.reshape(c["shape"]["lens"])
        idx = np.int32(c["indices"])
        idx = idx.reshape(c["indices_lens"]) if c["indices_lens"] is not None else idx.reshape(())
        got = orc.gather(data, idx, c["axis"])
        assert got.flatten().tolist() == [float(v) for v in c["gold"]], c["name"]
        assert np.array_equal(got, np.take(data, idx, axis=c["axis"]))


def test_binary_and_unary_are_the_ieee_and_libm_operations():
    rng = np.random.default_rng(2)
    a = rng.normal(0, 2, 1000).astype(np.float32)
    b = rng.uniform(0.5, 3, 1000).astype(np.float32)
    assert np.array_equal(orc.binary_f32("add", a, b), a + b)
    assert np.array_equal(orc.binary_f32("sub", a, b), a - b)
    assert np.array_equal(orc.binary_f32("mul", a, b), a * b)
    assert np.array_equal(orc.binary_f32("div", a, b), a / b)
    assert np.array_equal(orc.unary_f32("sqrt", b), np.sqrt(b))
    assert np.array_equal(orc.unary_f32("rsqrt", b), np.float32(1) / np.sqrt(b))
    assert np.array_equal(orc.unary_f32("neg", a), -a)
    erf = np.float32([math.erf(float(v)) for v in a])
    assert np.allclose(orc.unary_f32("erf", a), erf, rtol=3e-7, atol=1e-7)
    assert np.allclose(orc.unary_f32("exp", a), np.exp(a.astype(np.float64)), rtol=3e-7)
    assert np.allclose(orc.unary_f32("tanh", a), np.tanh(a.astype(np.float64)), rtol=3e-7, atol=1e-7)
    # the reference's own erf samples (test/ref/erf.cpp:38)
    x = np.float32([0.73785057, 1.58165966, -0.43597795, -0.01677432])
    assert np.allclose(orc.unary_f32("erf", x), [math.erf(float(v)) for v in x], rtol=3e-7)
