"""Seeded sweep of pointwise operators over arbitrarily permuted (and narrowed) views against
numpy: sizes around the transpose tiles' edges (multiples of 4 and not), 2 to 4 dims, copy,
scaled add, and two- and three-operand expressions.  Pure fp32 arithmetic, so bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32
SIZES = [1, 2, 3, 4, 8, 12, 16, 20, 36, 64, 68, 100, 128, 132, 200, 256, 260]


@pytest.mark.parametrize("chunk", range(4))
def test_permuted_views_against_numpy(cl, chunk):
    rs = np.random.RandomState(2025 + chunk)
    for it in range(40):
        nd = int(rs.choice([2, 3, 4]))
        shape = [int(rs.choice(SIZES)) for _ in range(nd)]
        while np.prod(shape) > 2_000_000:
            d = int(rs.randint(nd))
            shape[d] = max(1, shape[d] // 2)
        perm = [int(p) for p in rs.permutation(nd)]
        a = rs.standard_normal(shape).astype(F)
        b = rs.standard_normal([shape[p] for p in perm]).astype(F)          # b is stored permuted
        c = rs.standard_normal(shape).astype(F)
        A, Bp = cl.ClTensor(a), cl.ClTensor(b)
        Bv = Bp.permute(*[perm.index(i) + 1 for i in range(nd)])             # b seen with a's shape
        bv = b.transpose([perm.index(i) for i in range(nd)])
        assert Bv.size() == tuple(shape)
        off = int(rs.choice([0, 0, 1, 4]))
        if off and shape[-1] > off + 1:
            A2, a2 = A.narrow(nd, off + 1, shape[-1] - off), a[..., off:]
            B2, b2 = Bv.narrow(nd, off + 1, shape[-1] - off), bv[..., off:]
            c2 = np.ascontiguousarray(c[..., off:])
        else:
            A2, a2, B2, b2, c2 = A, a, Bv, bv, c
        C2 = cl.ClTensor(c2)
        kind = int(rs.randint(4))
        what = f"chunk {chunk} case {it}: shape {shape} perm {perm} offset {off} kind {kind}"
        if kind == 0:
            got, want = cl.ClTensor(*a2.shape).copy(B2).float(), b2
        elif kind == 1:
            want = a2 + F(0.5) * b2
            got = A2.add(0.5, B2).float()
        elif kind == 2:
            want = (a2 * b2 + c2).astype(F)
            got = A2.map2_on_gpu(B2, C2, "x = x*y + z").float()
        else:
            want = (c2 * F(2) + b2).astype(F)
            got = C2.map_on_gpu(B2, "x = x*2 + y").float()
        assert np.array_equal(got, want), what
        assert np.array_equal(Bp.float(), b), what + " (input modified)"
