"""dot, addmv, addr (and the THClBlas-level gemv / ger they sit on) through the
C ABI against fp64 numpy (oracle/catalogue.py).  Tolerance 1e-5 relative to the
result's scale for the sums (fp64 accumulation on the device), bit-exact for
the small-integer cases of the reference's own tests."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import catalogue as cat
from gpu_util import Pair

pytestmark = pytest.mark.gpu
F = np.float32


def _close(got, want, tol=1e-5):
    want = np.asarray(want, dtype=np.float64)
    scale = max(float(np.sqrt(np.mean(want ** 2))), 1e-30)
    assert got.shape == want.shape
    assert np.max(np.abs(got.astype(np.float64) - want)) / scale < tol


def test_reference_integer_matrices(cl):
    A = cl.ClTensor(np.array([[1, 2, -1], [3, 4, 0]], dtype=F))
    B = np.array([[0, 1], [1, 2], [4, 5]], dtype=F)
    assert cl.mv(A, cl.ClTensor(B[:, 0].copy())).float().tolist() == [-2.0, 4.0]
    assert cl.mv(A, cl.ClTensor(B[:, 1].copy())).float().tolist() == [0.0, 11.0]
    assert cl.ClTensor(np.array([1, 2, 3], dtype=F)).dot(cl.ClTensor(np.array([4, -5, 6], dtype=F))) == 12.0
    assert cl.ger(cl.ClTensor(np.array([1, 2], dtype=F)), cl.ClTensor(np.array([3, 4, 5], dtype=F))).float().tolist() == \
        [[3, 4, 5], [6, 8, 10]]


@pytest.mark.parametrize("n", [1, 3, 64, 1023, 4099, 1 << 20, (1 << 22) + 5])
def test_dot_lengths_and_views(cl, n):
    a, b = oracle.uniform(71, n), oracle.uniform(72, n)
    got = cl.ClTensor(a).dot(cl.ClTensor(b))
    want = float(cat.dot(a, b))
    assert abs(got - want) <= 1e-5 * max(abs(want), np.sqrt(n) * 1e-2)
    if n >= 64:
        pa = Pair(cl, a, 1, (n // 2,), (2,))                 # stride-2 view with an odd offset
        pb = Pair(cl, b, 0, (n // 2,), (1,))
        want = float(cat.dot(pa.view.gather(), pb.view.gather()))
        assert abs(pa.dev.dot(pb.dev) - want) <= 1e-5 * max(abs(want), np.sqrt(n) * 1e-2)
    with pytest.raises(cl.ClError):
        cl.ClTensor(a).dot(cl.ClTensor(n + 1))
    if n >= 4096 and n % 64 == 0:
        # both operands transposed alike: multiplied where they lie; one transposed, one not: through dense copies
        qa, qb = Pair.dense(cl, a.reshape(64, n // 64)).transpose(0, 1), Pair.dense(cl, b.reshape(64, n // 64)).transpose(0, 1)
        want = float(cat.dot(qa.view.gather(), qb.view.gather()))
        assert abs(qa.dev.dot(qb.dev) - want) <= 1e-5 * max(abs(want), np.sqrt(n) * 1e-2)
        qc = Pair.dense(cl, b.reshape(n // 64, 64))
        want = float(cat.dot(qa.view.gather(), qc.view.gather()))
        assert abs(qa.dev.dot(qc.dev) - want) <= 1e-5 * max(abs(want), np.sqrt(n) * 1e-2)


def test_blas_dot_on_storage_addresses(cl):
    """THClBlas_dot takes what storage->wrapper holds plus an offset and an increment per operand
    (src/lib/THClBlas.cpp:149-213)."""
    import ctypes as C
    lib, st = cl.state().lib, cl.state().ptr
    lib.THClBlas_dot.restype = C.c_float
    lib.THClTensor_wrapper.restype = C.c_void_p
    a, b = oracle.uniform(86, 5000), oracle.uniform(87, 5000)
    A, B = cl.ClTensor(a), cl.ClTensor(b)
    wa, wb = C.c_void_p(lib.THClTensor_wrapper(st, A._h)), C.c_void_p(lib.THClTensor_wrapper(st, B._h))
    L = C.c_long
    for n, xo, ix, yo, iy in ((5000, 0, 1, 0, 1), (1000, 3, 2, 7, 4), (1, 4999, 9, 4999, 9), (0, 0, 1, 0, 1)):
        got = lib.THClBlas_dot(st, L(n), wa, L(xo), L(ix), wb, L(yo), L(iy))
        cl.state().check()
        if n == 1:
            ix = iy = 1
        want = float(cat.dot(a[xo:xo + n * ix:ix], b[yo:yo + n * iy:iy])) if n else 0.0
        assert abs(got - want) <= 1e-5 * max(abs(want), 1e-2), (n, xo, ix, yo, iy, got, want)


@pytest.mark.parametrize("rows,cols", [(1, 1), (2, 3), (7, 130), (130, 7), (64, 64), (300, 1000), (1000, 300), (4096, 33),
                                       (33, 4096), (5, 70000), (70000, 5), (2048, 2048),
                                       # few long lines (cut over blocks), lines of 1..16 elements (a thread each), fewer than
                                       # 64 units of outputs (spare lanes take further columns)
                                       (3, 300001), (300001, 3), (4, 1 << 20), (1 << 20, 4), (16, 100000), (100000, 16),
                                       (40, 50000), (50000, 40), (1, 1 << 20), (1 << 20, 1)])
def test_addmv_layouts(cl, rows, cols):
    m = oracle.normal(73, rows * cols).reshape(rows, cols)
    v, t = oracle.normal(74, cols), oracle.normal(75, rows)
    M, V, T = cl.ClTensor(m), cl.ClTensor(v), cl.ClTensor(t)
    r = cl.ClTensor().addmv(0.5, T, 2.0, M, V)               # row-major matrix: the 't' kernel
    _close(r.float(), cat.addmv(0.5, t, 2.0, m, v))
    Mt = cl.ClTensor(np.ascontiguousarray(m.T)).t()          # same matrix stored column-major: the 'n' kernel
    assert Mt.size() == (rows, cols) and Mt.stride()[0] == 1
    r2 = cl.ClTensor().addmv(0.5, T, 2.0, Mt, V)
    _close(r2.float(), cat.addmv(0.5, t, 2.0, m, v))
    T2 = cl.ClTensor(t)
    T2.addmv(M, V)                                           # in place, beta = alpha = 1
    _close(T2.float(), cat.addmv(1.0, t, 1.0, m, v))
    _close(cl.mv(M, V).float(), cat.addmv(0.0, np.zeros(rows), 1.0, m, v))
    if rows >= 4 and cols >= 4:                              # neither stride is 1: dense copy, then 't'
        big = Pair.dense(cl, oracle.normal(76, rows * cols * 4).reshape(rows * 2, cols * 2))
        sub = big.step(0, 2).step(1, 2)
        r3 = cl.ClTensor().addmv(1.0, T, 1.0, sub.dev, V)
        _close(r3.float(), cat.addmv(1.0, t, 1.0, sub.view.gather(), v))
        # strided vector and result
        vv = Pair(cl, oracle.normal(77, cols * 3), 1, (cols,), (3,))
        rr = Pair(cl, np.zeros(rows * 2, dtype=F), 0, (rows,), (2,))
        rr.dev.addmv(0.0, rr.dev, 1.0, M, vv.dev)
        _close(rr.dev.float(), cat.addmv(0.0, np.zeros(rows), 1.0, m, vv.view.gather()))


@pytest.mark.parametrize("rows,cols,pitch,first", [(300, 256, 259, 1), (300, 255, 259, 2), (64, 4100, 4101, 1), (64, 4099, 4101, 0),
                                                   (2000, 64, 67, 3), (2000, 61, 67, 3), (16, 30001, 30004, 1)])
def test_addmv_on_rows_that_start_at_odd_elements(cl, rows, cols, pitch, first):
    """A block cut out of a wider matrix, row- and column-major: lines that start at any element, of any length (units
    of four read without alignment, then the last elements one by one)."""
    big = oracle.normal(88, rows * pitch).reshape(rows, pitch)
    m = big[:, first:first + cols]
    v, t = oracle.normal(89, cols), oracle.normal(90, rows)
    M = cl.ClTensor(big).narrow(2, first + 1, cols)
    V, T = cl.ClTensor(v), cl.ClTensor(t)
    _close(cl.ClTensor().addmv(0.5, T, 2.0, M, V).float(), cat.addmv(0.5, t, 2.0, m, v))
    # the transposed product walks the same memory along the other dim
    _close(cl.ClTensor().addmv(0.5, V, 2.0, M.t(), T).float(), cat.addmv(0.5, v, 2.0, np.ascontiguousarray(m.T), t))


def test_addmv_beta_zero_ignores_old_contents_and_checks_shapes(cl):
    m = oracle.normal(78, 40 * 30).reshape(40, 30)
    v = oracle.normal(79, 30)
    t = np.full(40, np.nan, dtype=F)                          # BLAS: beta == 0 means y is not read
    r = cl.ClTensor().addmv(0.0, cl.ClTensor(t), 1.0, cl.ClTensor(m), cl.ClTensor(v))
    _close(r.float(), cat.addmv(0.0, np.zeros(40), 1.0, m, v))
    with pytest.raises(cl.ClError):
        cl.ClTensor().addmv(cl.ClTensor(t), cl.ClTensor(m), cl.ClTensor(31))
    with pytest.raises(cl.ClError):
        cl.ClTensor().addmv(cl.ClTensor(39), cl.ClTensor(m), cl.ClTensor(v))
    with pytest.raises(cl.ClError):
        cl.ClTensor().addmv(cl.ClTensor(t), cl.ClTensor(v), cl.ClTensor(v))


def test_addr_kernel_and_generic_path_agree_bit_for_bit(cl):
    """A matrix with unit stride along one dim, 16-byte aligned, takes the rank-1 kernel; the same values in a
    view that starts 4 bytes off a 16-byte boundary take the pointwise engine.  Same association, same bits."""
    rows, cols = 1000, 1000
    t = oracle.normal(83, rows * cols).reshape(rows, cols)
    a, b = oracle.normal(84, rows), oracle.normal(85, cols)
    A, B = cl.ClTensor(a), cl.ClTensor(b)
    wide = np.zeros((rows, cols + 4), dtype=F)
    wide[:, 1:cols + 1] = t
    for beta, alpha in ((1.0, 0.5), (0.9, -1.25)):
        fast = cl.ClTensor(t)
        fast.addr(beta, alpha, A, B)
        slow = cl.ClTensor(wide).narrow(2, 2, cols)
        slow.addr(beta, alpha, A, B)
        assert np.array_equal(fast.float().view(np.uint32), slow.float().view(np.uint32)), (beta, alpha)
        # column-major: the transposed view of a (cols x rows) matrix
        fast_t = cl.ClTensor(np.ascontiguousarray(t.T)).t()
        fast_t.addr(beta, alpha, A, B)
        assert np.array_equal(fast_t.float().view(np.uint32), slow.float().view(np.uint32)), (beta, alpha, "column-major")


@pytest.mark.parametrize("rows,cols", [(1, 1), (2, 3), (130, 70), (64, 256), (1000, 1000), (5, 50000), (50000, 5)])
def test_addr_layouts(cl, rows, cols):
    t = oracle.normal(80, rows * cols).reshape(rows, cols)
    a, b = oracle.normal(81, rows), oracle.normal(82, cols)
    T, A, B = cl.ClTensor(t), cl.ClTensor(a), cl.ClTensor(b)
    r = cl.ClTensor().addr(0.5, T, 2.0, A, B)
    _close(r.float(), cat.addr(0.5, t, 2.0, a, b))
    T2 = cl.ClTensor(t)
    T2.addr(A, B)                                            # in place, beta = alpha = 1
    _close(T2.float(), cat.addr(1.0, t, 1.0, a, b))
    _close(cl.ger(A, B).float(), cat.addr(0.0, np.zeros((rows, cols)), 1.0, a, b))
    Tt = Pair.dense(cl, np.ascontiguousarray(t.T)).transpose(0, 1)    # column-major result
    Tt.dev.addr(1.0, 3.0, A, B)
    _close(Tt.dev.float(), cat.addr(1.0, t, 3.0, a, b))
    if rows >= 2:
        aa = Pair(cl, oracle.normal(83, rows * 2 + 1), 1, (rows,), (2,))   # strided vector
        T3 = cl.ClTensor(t)
        T3.addr(1.0, 1.0, aa.dev, B)
        _close(T3.float(), cat.addr(1.0, t, 1.0, aa.view.gather(), b))
    with pytest.raises(cl.ClError):
        cl.ClTensor().addr(T, A, cl.ClTensor(cols + 1))


def test_blas_level_entry_points(cl):
    """THClBlas_gemv / ger with explicit leading dimensions, as the reference's
    tensor-level code calls them (src/lib/THClTensorMathBlas.cpp:62-104,241-276)."""
    from cltorch_amd.tensor import _call
    m, n, lda = 37, 29, 48
    store = oracle.normal(84, lda * n)
    a = cl.ClTensor(store)
    x, y = oracle.normal(85, n), oracle.normal(86, m)
    X, Y = cl.ClTensor(x), cl.ClTensor(y)
    _call("THClBlas_gemv", C.c_char(b"n"), C.c_long(m), C.c_long(n), C.c_float(1.5), a._h, C.c_long(lda), X._h, C.c_long(1),
                      C.c_float(0.25), Y._h, C.c_long(1))
    A = store.reshape(n, lda)[:, :m].T.astype(np.float64)     # column-major m x n
    _close(Y.float(), 0.25 * y + 1.5 * (A @ x))
    xt, yt = oracle.normal(87, m), oracle.normal(88, n)
    XT, YT = cl.ClTensor(xt), cl.ClTensor(yt)
    _call("THClBlas_gemv", C.c_char(b"t"), C.c_long(m), C.c_long(n), C.c_float(1.0), a._h, C.c_long(lda), XT._h, C.c_long(1),
                      C.c_float(1.0), YT._h, C.c_long(1))
    _close(YT.float(), yt + A.T @ xt)
    _call("THClBlas_ger", C.c_long(m), C.c_long(n), C.c_float(2.0), XT._h, C.c_long(1), X._h, C.c_long(1), a._h, C.c_long(lda))
    want = store.reshape(n, lda).astype(np.float64).copy()
    want[:, :m] += 2.0 * np.outer(x, xt)
    _close(a.float().reshape(n, lda), want)                  # padding rows beyond m untouched
    assert np.array_equal(a.float().reshape(n, lda)[:, m:], store.reshape(n, lda)[:, m:])
