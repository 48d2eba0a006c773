"""The rest of the pointwise operator catalogue through the C ABI, against the
numpy restatement in oracle/catalogue.py.  Exact operators compare bit for bit;
transcendental ones within 1e-4 absolute / 2e-6 relative, inside the tolerance the reference's
own tests use (src/test/unit_tensor.lua:73-93)."""
import numpy as np
import pytest

import oracle
from oracle import catalogue as cat
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32
N = 70001


def _close(got, want, what):
    both_nan = np.isnan(got) & np.isnan(want)
    both_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    ok = both_nan | both_inf | (np.abs(got - want) <= 1e-4 + 2e-6 * np.abs(want))
    assert ok.all(), f"{what}: worst {np.nanmax(np.abs(got - want)[~(both_nan | both_inf)])} at {np.argmin(ok)}"


@pytest.mark.parametrize("name,lo,hi", [("log1p", -0.9, 50.0), ("cos", -20.0, 20.0), ("sin", -20.0, 20.0), ("tan", -1.5, 1.5),
                                        ("acos", -1.0, 1.0), ("asin", -1.0, 1.0), ("atan", -100.0, 100.0),
                                        ("cosh", -8.0, 8.0), ("sinh", -8.0, 8.0)])
def test_unary_transcendental(cl, name, lo, hi):
    x = oracle.uniform(41, N, lo, hi)
    X = cl.ClTensor(x)
    R = cl.ClTensor()
    getattr(R, name)(X)                                   # two-tensor form resizes the result
    assert R.size() == (N,)
    want = cat.unary(name, x)
    scale = np.maximum(1.0, np.abs(want))
    _close(R.float() / scale, want / scale, name)
    getattr(X, name)()                                    # in place: same kernel family, one operand
    _close(X.float() / scale, want / scale, name + " in place")


def test_round_and_sign_are_exact(cl):
    x = oracle.uniform(42, N, -40.0, 40.0)
    x[:11] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.49999997, -0.49999997, 0.0, -0.0, 8388609.0]
    x[11:14] = [np.nan, np.inf, -np.inf]
    for name in ("round", "sign"):
        R = cl.ClTensor()
        getattr(R, name)(cl.ClTensor(x))
        assert_bit_equal(R.float(), cat.unary(name, x), name)
    p = Pair.dense(cl, x[:60000].reshape(200, 300)).transpose(0, 1)   # strided in place
    p.dev.round()
    assert_bit_equal(p.dev.float(), cat.unary("round", p.view.gather()), "round on a transposed view")


def test_pow_forms(cl):
    x = oracle.uniform(43, N, 0.1, 3.0)
    xs = oracle.uniform(44, N, -3.0, 3.0)
    for v in (2.0, 3.0, -2.0, 0.0, 7.0):                 # integer-valued: repeated multiplication, exact
        R = cl.ClTensor().pow(cl.ClTensor(xs), v)
        assert_bit_equal(R.float(), cat.pow_value(xs, v), f"pow {v}")
    for v in (0.5, 2.5, -1.25):
        R = cl.ClTensor().pow(cl.ClTensor(x), v)
        want = cat.pow_value(x, v)
        assert np.allclose(R.float(), want, rtol=3e-6, atol=0), f"pow {v}"
    X = cl.ClTensor(x)
    X.pow(2.0)
    assert_bit_equal(X.float(), (x * x).astype(F), "in-place square")
    R = cl.ClTensor().pow(2.0, cl.ClTensor(xs))            # value ^ tensor
    assert np.allclose(R.float(), cat.tpow(2.0, xs), rtol=3e-6)
    e = oracle.uniform(45, N, -2.0, 2.0)
    R = cl.ClTensor().cpow(cl.ClTensor(x), cl.ClTensor(e))
    assert np.allclose(R.float(), cat.cpow(x, e), rtol=3e-6)
    X = cl.ClTensor(x)
    X.cpow(cl.ClTensor(e))
    assert np.allclose(X.float(), cat.cpow(x, e), rtol=3e-6)


def test_clamp_cmax_cmin_atan2(cl):
    x, y = oracle.uniform(46, N, -2.0, 2.0), oracle.uniform(47, N, -2.0, 2.0)
    X, Y = cl.ClTensor(x), cl.ClTensor(y)
    assert_bit_equal(cl.ClTensor().clamp(X, -0.5, 0.75).float(), cat.clamp(x, -0.5, 0.75), "clamp")
    Z = cl.ClTensor(x)
    Z.clamp(-0.25, 0.25)
    assert_bit_equal(Z.float(), cat.clamp(x, -0.25, 0.25), "clamp in place")
    assert_bit_equal(cl.ClTensor().cmax(X, Y).float(), cat.cmax(x, y), "cmax")
    assert_bit_equal(cl.ClTensor().cmin(X, Y).float(), cat.cmin(x, y), "cmin")
    assert_bit_equal(cl.ClTensor().cmax(X, 0.5).float(), cat.cmax(x, 0.5), "cmaxValue")
    assert_bit_equal(cl.ClTensor().cmin(X, 0.5).float(), cat.cmin(x, 0.5), "cminValue")
    Z = cl.ClTensor(x)
    Z.cmax(Y)
    assert_bit_equal(Z.float(), cat.cmax(x, y), "cmax in place")
    Z.cmin(0.0)
    assert_bit_equal(Z.float(), cat.cmin(cat.cmax(x, y), 0.0), "cminValue in place")
    got = cl.ClTensor().atan2(X, Y).float()
    _close(got, cat.atan2(x, y), "atan2")
    with pytest.raises(cl.ClError):
        cl.ClTensor().atan2(X, cl.ClTensor(5))


@pytest.mark.parametrize("name", ["lt", "gt", "le", "ge", "eq", "ne"])
def test_comparisons(cl, name):
    x = np.round(oracle.uniform(48, N, -4.0, 4.0)).astype(F)      # many exact ties
    y = np.round(oracle.uniform(49, N, -4.0, 4.0)).astype(F)
    x[:3] = [np.nan, 1.0, np.nan]
    y[:3] = [1.0, np.nan, np.nan]
    X, Y = cl.ClTensor(x), cl.ClTensor(y)
    assert_bit_equal(getattr(X, name)(1.0).float(), cat.compare(name, x, 1.0), name + "Value")
    assert_bit_equal(getattr(X, name)(Y).float(), cat.compare(name, x, y), name + "Tensor")
    pt = cl.ClTensor()
    pt.max(Y.narrow(1, 4, 100))                           # a device-side scalar
    assert pt.nDimension() == 0
    assert_bit_equal(getattr(X, name)(pt).float(), cat.compare(name, x, F(pt.s())), name + "PointTensor")
    res = cl.ClTensor(3)                                  # an existing result is resized
    getattr(res, name)(X, Y)
    assert res.size() == (N,)
    # strided operands
    px, py = Pair.dense(cl, x[:60000].reshape(200, 300)), Pair.dense(cl, y[:60000].reshape(300, 200))
    got = getattr(px.dev, name)(py.transpose(0, 1).dev)
    assert_bit_equal(got.float(), cat.compare(name, px.view.gather(), py.transpose(0, 1).view.gather()), name + " strided")
    with pytest.raises(cl.ClError):
        getattr(X, name)(cl.ClTensor(5))


def test_masked_fill(cl):
    x = oracle.uniform(50, N)
    m = (oracle.uniform(51, N) > 0.3).astype(F)
    m[:4] = [0.0, -0.0, 2.0, -1.0]                         # any non-zero selects
    X = cl.ClTensor(x)
    X.maskedFill(cl.ClTensor(m), 7.5)
    assert_bit_equal(X.float(), cat.masked_fill(x, m, 7.5), "maskedFill")
    p = Pair.dense(cl, x[:60000].reshape(200, 300)).transpose(0, 1)
    pm = Pair.dense(cl, m[:60000].reshape(300, 200))
    p.dev.maskedFill(pm.dev, -1.0)
    assert_bit_equal(p.dev.float(), cat.masked_fill(p.view.gather(), pm.view.gather(), -1.0), "maskedFill strided")
    with pytest.raises(cl.ClError):
        X.maskedFill(cl.ClTensor(5), 1.0)
