"""Seeded sweep of gather, scatter, scatterFill, indexFill, indexCopy and the masked operators over
arbitrarily permuted views against numpy, with masks that select nothing or everything among them."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32
SIZES = [1, 2, 3, 4, 7, 16, 33, 64, 100, 257, 1024]


def _permuted(cl, rs, shape):
    nd = len(shape)
    perm = [int(p) for p in rs.permutation(nd)]
    b = rs.standard_normal([shape[p] for p in perm]).astype(F)
    back = [perm.index(i) for i in range(nd)]
    return cl.ClTensor(b).permute(*[p + 1 for p in back]), b.transpose(back)


@pytest.mark.parametrize("chunk", range(3))
def test_permuted_index_and_masked_operators_against_numpy(cl, chunk):
    rs = np.random.RandomState(501 + chunk)
    for it in range(25):
        nd = int(rs.choice([2, 3]))
        shape = [int(rs.choice(SIZES)) for _ in range(nd)]
        while np.prod(shape) > 500_000:
            d = int(rs.randint(nd))
            shape[d] = max(1, shape[d] // 2)
        dim = int(rs.randint(nd))
        what = f"chunk {chunk} case {it}: shape {shape} dim {dim + 1}"
        along = lambda part: tuple(slice(None) if d != dim else part for d in range(nd))

        S, s = _permuted(cl, rs, shape)
        ishape = list(shape)
        ishape[dim] = int(rs.randint(1, 2 * shape[dim] + 1))
        idx = rs.randint(1, shape[dim] + 1, size=ishape)
        got = S.gather(dim + 1, cl.ClTensor(idx.astype(F))).float()
        assert np.array_equal(got, np.take_along_axis(s, idx - 1, axis=dim)), what + " gather"

        # scatter targets are a permutation along every line, so the result does not depend on order
        base, want = _permuted(cl, rs, shape)
        want = want.copy()
        pidx = np.argsort(rs.uniform(size=shape), axis=dim) + 1
        src, s0 = _permuted(cl, rs, shape)
        base.scatter(dim + 1, cl.ClTensor(pidx.astype(F)), src)
        np.put_along_axis(want, pidx - 1, s0, axis=dim)
        assert np.array_equal(base.float(), want), what + " scatter"
        base.scatter(dim + 1, cl.ClTensor(pidx.astype(F)), 2.5)
        np.put_along_axis(want, pidx - 1, F(2.5), axis=dim)
        assert np.array_equal(base.float(), want), what + " scatterFill"

        k = int(rs.randint(1, shape[dim] + 1))
        sel = rs.permutation(shape[dim])[:k] + 1
        T, w = _permuted(cl, rs, shape)
        w = w.copy()
        T.indexFill(dim + 1, sel.astype(np.int64), -3.0)
        w[along(sel - 1)] = -3
        assert np.array_equal(T.float(), w), what + " indexFill"
        cshape = list(shape)
        cshape[dim] = k
        C, c0 = _permuted(cl, rs, cshape)
        T.indexCopy(dim + 1, sel.astype(np.int64), C)
        w[along(sel - 1)] = c0
        assert np.array_equal(T.float(), w), what + " indexCopy"

        density = [0.0, 1.0, rs.uniform(), rs.uniform()][it % 4]
        mask = (rs.uniform(size=shape) < density).astype(F)
        M = cl.ClTensor(mask)
        count = int((mask != 0).sum())
        picked = T.maskedSelect(M)
        assert picked.nElement() == count, what + " maskedSelect count"
        assert np.array_equal(picked.float(), w[mask != 0]), what + " maskedSelect"
        T.maskedFill(M, 9.0)
        w[mask != 0] = 9
        assert np.array_equal(T.float(), w), what + " maskedFill"
        vals = rs.standard_normal(count + 3).astype(F)
        T.maskedCopy(M, cl.ClTensor(vals))
        w[mask != 0] = vals[:count]
        assert np.array_equal(T.float(), w), what + " maskedCopy"
