"""Seeded sweep of reductions along a dim (sum, max/min with positions), cumsum, whole-tensor
reductions, the 2-norm and index selection over arbitrarily permuted views against numpy."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32
SIZES = [1, 2, 3, 4, 5, 8, 16, 17, 33, 64, 100, 128, 257, 1000, 1024, 4100]


@pytest.mark.parametrize("chunk", range(4))
def test_permuted_reductions_against_numpy(cl, chunk):
    rs = np.random.RandomState(77 + chunk)
    for it in range(30):
        nd = int(rs.choice([1, 2, 3, 4]))
        shape = [int(rs.choice(SIZES)) for _ in range(nd)]
        while np.prod(shape) > 2_000_000:
            d = int(rs.randint(nd))
            shape[d] = max(1, shape[d] // 2)
        perm = [int(p) for p in rs.permutation(nd)]
        b = rs.standard_normal([shape[p] for p in perm]).astype(F)
        Bv = cl.ClTensor(b).permute(*[perm.index(i) + 1 for i in range(nd)])
        bv = b.transpose([perm.index(i) for i in range(nd)])
        dim = int(rs.randint(nd))
        b64 = bv.astype(np.float64)
        what = f"chunk {chunk} case {it}: shape {shape} perm {perm} dim {dim + 1}"
        slack = 1e-4 * np.sqrt(shape[dim])
        assert np.allclose(Bv.sum(dim + 1).float(), b64.sum(axis=dim, keepdims=True), rtol=1e-5, atol=slack), what
        v, i = Bv.max(dim + 1)
        assert np.array_equal(v.float(), bv.max(axis=dim, keepdims=True)), what
        assert np.array_equal(i.float(), np.expand_dims(bv.argmax(axis=dim), dim) + 1), what
        v, i = Bv.min(dim + 1)
        assert np.array_equal(v.float(), bv.min(axis=dim, keepdims=True)), what
        assert np.array_equal(i.float(), np.expand_dims(bv.argmin(axis=dim), dim) + 1), what
        assert np.allclose(Bv.cumsum(dim + 1).float(), np.cumsum(b64, axis=dim), rtol=1e-5, atol=slack), what
        assert abs(Bv.sum() - b64.sum()) <= 1e-5 * np.abs(b64).sum() + 1e-6, what
        assert Bv.max() == bv.max() and Bv.min() == bv.min(), what
        assert np.isclose(Bv.norm(2), np.sqrt((b64 ** 2).sum()), rtol=1e-5), what
        idx = rs.randint(1, shape[dim] + 1, size=int(rs.randint(1, 2 * shape[dim] + 2)))
        assert np.array_equal(Bv.index(dim + 1, idx.astype(np.int64)).float(), np.take(bv, idx - 1, axis=dim)), what
