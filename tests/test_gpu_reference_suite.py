"""The reference's own unit tests that have no direct counterpart elsewhere in this suite,
restated against the Python mirror (src/test/unit_tensor.lua, line numbers at each test).
Where the reference compares with the CPU FloatTensor result, the expected values here are
numpy fp32 ones."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32


def test_equals(cl):                                   # unit_tensor.lua:202-220
    c = cl.ClTensor([[3, 5, -2], [2.1, 2.2, 3.9]])
    d = cl.ClTensor([[3, 5, -2], [2.1, 2.2, 3.9]])
    e = cl.ClTensor([[3, 5, -2], [2.1, 2.4, 3.9]])
    assert np.array_equal(c.float(), d.float()) and not np.array_equal(c.float(), e.float())


def test_matrixwide(cl):                               # unit_tensor.lua:488-496
    a = np.array([[3, 2, 4], [9, 7, 5]], dtype=F)
    c = cl.ClTensor(a)
    assert c.max() == 9 and c.min() == 2 and c.sum() == 30
    assert np.array_equal(c.sum(1).float(), a.sum(axis=0, keepdims=True))
    assert np.array_equal(c.sum(2).float(), a.sum(axis=1, keepdims=True))


def test_intpower_and_powerofneg(cl):                  # unit_tensor.lua:506-520
    a = np.array([[3.3, -2.2, 0], [9, 7, 5]], dtype=F)
    got = cl.ClTensor().pow(cl.ClTensor(a), 2).float()
    assert np.allclose(got, a * a, rtol=1e-6, atol=0)
    got = cl.ClTensor().pow(cl.ClTensor(a), 2.4).float()
    with np.errstate(invalid="ignore"):
        want = np.power(a, F(2.4))
    assert np.isnan(got[0, 1]) and np.isnan(want[0, 1])          # a negative base to a fractional power
    ok = ~np.isnan(want)
    assert np.allclose(got[ok], want[ok], rtol=2e-6, atol=1e-6)


def test_addcdivshape(cl):                             # unit_tensor.lua:1054-1060
    rng = np.random.RandomState(3)
    a0 = rng.uniform(0.1, 1, (3, 2, 4)).astype(F)
    b0 = rng.uniform(0.1, 1, 24).astype(F)
    a, b = cl.ClTensor(a0), cl.ClTensor(b0)
    assert a.nDimension() == 3
    a.addcdiv(1, b, b)
    assert a.nDimension() == 3 and a.size() == (3, 2, 4)
    assert np.array_equal(a.float(), (a0 + (b0 / b0).reshape(3, 2, 4)).astype(F))


def test_get(cl):                                      # unit_tensor.lua:1062-1072
    from cltorch_amd.tensor import _call
    import ctypes as C
    acl = cl.ClTensor(20, 5, 14).zero()
    _call("THClTensor_set3d", acl._h, 14, 1, 11, C.c_float(250))
    _call("THClTensor_set3d", acl._h, 14, 1, 13, C.c_float(255))
    cl.state().lib.THClTensor_get3d.restype = C.c_float
    assert _call("THClTensor_get3d", acl._h, 14, 1, 11) == 250
    assert _call("THClTensor_get3d", acl._h, 14, 1, 13) == 255
    assert acl.sum() == 505


@pytest.mark.parametrize("op", ["lt", "gt", "le", "ge", "eq", "ne"])
def test_inplace_and_outplace_compare(cl, op):         # unit_tensor.lua:222-306
    a = np.array([[4, 2, -1], [3.1, 1.2, 4.9]], dtype=F)
    b = np.array([[3, 5, -2], [2.1, 2.2, 3.9]], dtype=F)
    fn = {"lt": np.less, "gt": np.greater, "le": np.less_equal, "ge": np.greater_equal, "eq": np.equal, "ne": np.not_equal}[op]
    A, B = cl.ClTensor(a), cl.ClTensor(b)
    assert np.array_equal(getattr(cl.ClTensor(), op)(A, B).float(), fn(a, b).astype(F))
    assert np.array_equal(getattr(cl.ClTensor(), op)(A, 3.0).float(), fn(a, F(3.0)).astype(F))
    r = getattr(A, op)(B)                              # the method form returns a new tensor and leaves a as it was
    assert np.array_equal(r.float(), fn(a, b).astype(F)) and np.array_equal(A.float(), a)
