"""Seeded sweep of addmm, addmv, addr and dot over random sizes, operand layouts (dense,
transposed, rows inside a wider buffer), strided vectors and alpha / beta against fp64."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32
SIZES = [1, 2, 3, 5, 16, 31, 64, 65, 100, 128, 130, 256, 300, 512, 1000, 2048, 4096]


def _view(cl, arr2d, transposed, pad):
    """A device tensor equal to arr2d, stored transposed and/or inside a wider buffer."""
    a = arr2d.T if transposed else arr2d
    r, c = a.shape
    big = np.zeros((r, c + pad), dtype=F)
    big[:, :c] = a
    t = cl.ClTensor(big)
    if pad:
        t = t.narrow(2, 1, c)
    return t.t() if transposed else t


def _rel(got, want):
    return float(np.max(np.abs(got - want)) / (np.sqrt(np.mean(want.astype(np.float64) ** 2)) + 1e-30))


@pytest.mark.parametrize("chunk", range(4))
def test_contractions_against_fp64(cl, chunk):
    rs = np.random.RandomState(99 + chunk)
    for it in range(25):
        M, N, K = (int(rs.choice(SIZES)) for _ in range(3))
        while M * N * K > 2e9 or M * K > 4e6 or K * N > 4e6 or M * N > 4e6:
            M, N, K = max(1, M // 2), max(1, N // 2), max(1, K // 2)
        a = (rs.standard_normal((M, K)) / np.sqrt(K)).astype(F)
        b = rs.standard_normal((K, N)).astype(F)
        c = rs.standard_normal((M, N)).astype(F)
        ta, tb, tc = (bool(rs.randint(2)) for _ in range(3))
        pa, pb, pc = (int(rs.choice([0, 0, 4, 7])) for _ in range(3))
        beta, alpha = float(rs.choice([0.0, 1.0, 0.5, -2.0])), float(rs.choice([1.0, 0.25, -1.5]))
        what = f"chunk {chunk} case {it}: {M}x{N}x{K} transposed {ta, tb, tc} pad {pa, pb, pc} beta {beta} alpha {alpha}"
        A, B, Cc = _view(cl, a, ta, pa), _view(cl, b, tb, pb), _view(cl, c, tc, pc)
        a64, b64, c64 = a.astype(np.float64), b.astype(np.float64), c.astype(np.float64)
        Cc.addmm(beta, alpha, A, B)
        assert _rel(Cc.float(), beta * c64 + alpha * (a64 @ b64)) < 1e-4, what
        x, y = rs.standard_normal(K).astype(F), rs.standard_normal(M).astype(F)
        step = int(rs.choice([1, 2, 3]))
        Xv = cl.ClTensor(np.repeat(x, step)).strided([K], [step], 1)
        Y = cl.ClTensor(y)
        Y.addmv(beta, alpha, A, Xv)
        assert _rel(Y.float(), beta * y.astype(np.float64) + alpha * (a64 @ x.astype(np.float64))) < 1e-4, what
        u, v = rs.standard_normal(M).astype(F), rs.standard_normal(N).astype(F)
        R = _view(cl, c, tc, pc)
        R.addr(beta, alpha, cl.ClTensor(u), cl.ClTensor(v))
        assert _rel(R.float(), beta * c64 + alpha * np.outer(u.astype(np.float64), v.astype(np.float64))) < 1e-5, what
        xx = float(x.astype(np.float64) @ x.astype(np.float64))
        assert abs(Xv.dot(cl.ClTensor(x)) - xx) <= 1e-5 * xx + 1e-6, what
