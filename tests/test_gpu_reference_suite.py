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


def test_basic_and_clone_text(cl):                     # unit_tensor.lua:164-199
    c = cl.ClTensor([7, 4, 5])
    assert str(c) == " 7\n 4\n 5\n[torch.ClTensor of size 3]\n"
    c = cl.ClTensor([[3, 1, 6], [2.1, 5.2, 3.9]])
    d = cl.ClTensor(2, 3).copy(c)
    want = " 3.0000  1.0000  6.0000\n 2.1000  5.2000  3.9000\n[torch.ClTensor of size 2x3]\n"
    assert str(c) == want and str(d) == want
    c = cl.ClTensor([[7, 4, 5], [3, 1, 4]])
    d = c.clone().fill(3)
    assert str(c) == " 7  4  5\n 3  1  4\n[torch.ClTensor of size 2x3]\n"          # the clone's fill left c alone
    assert str(d) == " 3  3  3\n 3  3  3\n[torch.ClTensor of size 2x3]\n"


C0 = np.array([[4, 2, -1], [3.1, 1.2, 4.9]], dtype=F)
D0 = np.array([[3, 5, -2], [2.1, 2.2, 3.9]], dtype=F)


def test_operators(cl):                                # unit_tensor.lua:349-375,401-405; src/TensorOperator.c
    c, d = cl.ClTensor(C0), cl.ClTensor(D0)
    v = F(3.4)
    assert np.array_equal((c + 3.4).float(), C0 + v) and np.array_equal((3.4 + c).float(), C0 + v)
    assert np.array_equal((c - 3.4).float(), C0 + (-v))
    assert np.array_equal((3.4 - c).float(), v + F(-1) * C0)
    assert np.array_equal((c * 3.4).float(), C0 * v) and np.array_equal((3.4 * c).float(), C0 * v)
    assert np.array_equal((c / 3.4).float(), C0 * F(1.0 / 3.4))       # a multiplication by the reciprocal
    assert np.array_equal((c + d).float(), C0 + D0) and np.array_equal((c - d).float(), C0 + F(-1) * D0)
    assert np.array_equal((-c).float(), -C0)
    assert np.array_equal(c.float(), C0) and np.array_equal(d.float(), D0)                # operands untouched
    # tensor * tensor by dimensions: dot, mv, mm
    a = cl.ClTensor([1, 2, 3]); b = cl.ClTensor([4, -5, 6])
    assert a * b == 12
    m = cl.ClTensor([[1, 2, -1], [3, 4, 0]])
    assert np.array_equal((m * a).float(), np.array([2, 11], dtype=F))
    n = cl.ClTensor([[0, 1], [1, 2], [4, 5]])
    assert np.array_equal((m * n).float(), np.array([[-2, 0], [4, 11]], dtype=F))
    with pytest.raises(cl.ClError):
        cl.ClTensor(2, 2, 2).zero() * m


def test_perelement(cl):                               # unit_tensor.lua:377-411
    c, d = cl.ClTensor(C0), cl.ClTensor(D0)
    assert np.array_equal(c.add(d).float(), C0 + D0)
    c = cl.ClTensor(C0)
    assert np.array_equal(c.cmul(d).float(), C0 * D0)
    c = cl.ClTensor(C0)
    assert np.array_equal(cl.ClTensor().clamp(c, 1.5, 4.5).float(), np.clip(C0, F(1.5), F(4.5)))


@pytest.mark.parametrize("name", ["add", "mul", "div", "pow", "lt", "le", "gt", "ge", "ne", "eq"])
def test_outplace_with_a_number(cl, name):             # unit_tensor.lua:337-347
    c = cl.ClTensor(C0)
    got = getattr(cl.ClTensor(), name)(c, 3.4).float()
    v = F(3.4)
    with np.errstate(invalid="ignore"):
        want = {"add": lambda: C0 + v, "mul": lambda: C0 * v, "div": lambda: C0 * F(1.0 / 3.4),
                "pow": lambda: np.power(C0, v), "lt": lambda: (C0 < v).astype(F), "le": lambda: (C0 <= v).astype(F),
                "gt": lambda: (C0 > v).astype(F), "ge": lambda: (C0 >= v).astype(F), "ne": lambda: (C0 != v).astype(F),
                "eq": lambda: (C0 == v).astype(F)}[name]()
    if name in ("pow", "div"):
        ok = ~np.isnan(want)
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.allclose(got[ok], want[ok], rtol=2e-6, atol=2e-4)
    else:
        assert np.array_equal(got, want)
    assert np.array_equal(c.float(), C0)
