"""Seeded differential testing of the apply planner: random shapes, random
chains of transpose / narrow / step views, one to three operands, fixed and
run-time compiled operators -- device result against the CPU oracle, bit for
bit, storages compared whole (so a stray write outside a view is caught)."""
import numpy as np
import pytest

import oracle
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32


def _random_view(rs, pair, min_elems=1):
    """A chain of view operations on a dense Pair."""
    p = pair
    for _ in range(rs.randint(0, 4)):
        nd = len(p.view.sizes)
        kind = rs.randint(0, 3)
        if kind == 0 and nd >= 2:
            a, b = rs.choice(nd, 2, replace=False)
            p = p.transpose(int(a), int(b))
        elif kind == 1:
            d = int(rs.randint(0, nd))
            n = p.view.sizes[d]
            if n > 1:
                first = int(rs.randint(0, n - 1))
                size = int(rs.randint(1, n - first + 1))
                p = p.narrow(d, first, size)
        else:
            d = int(rs.randint(0, nd))
            if p.view.sizes[d] > 2:
                p = p.step(d, int(rs.randint(2, 4)))
    return p


def _same_shape_view(rs, cl, shape, seed):
    """A view of exactly `shape` carved out of a larger random storage, by random means."""
    nd = len(shape)
    mode = rs.randint(0, 4)
    if mode == 0:      # dense
        return Pair.dense(cl, oracle.uniform(seed, int(np.prod(shape))).reshape(shape))
    if mode == 1:      # transposed storage
        perm = rs.permutation(nd)
        base = Pair.dense(cl, oracle.uniform(seed, int(np.prod(shape))).reshape([shape[i] for i in perm]))
        inv = np.argsort(perm)
        # bring dims back into order by transposes
        p, cur = base, list(perm)
        for d in range(nd):
            j = cur.index(d)
            if j != d:
                p = p.transpose(d, j)
                cur[d], cur[j] = cur[j], cur[d]
        assert tuple(p.view.sizes) == tuple(shape), (p.view.sizes, shape, inv)
        return p
    if mode == 2:      # narrowed out of a padded storage
        pad = [int(rs.randint(0, 4)) for _ in shape]
        big = Pair.dense(cl, oracle.uniform(seed, int(np.prod([s + 2 * q for s, q in zip(shape, pad)]))).reshape(
            [s + 2 * q for s, q in zip(shape, pad)]))
        p = big
        for d, q in enumerate(pad):
            p = p.narrow(d, q, shape[d])
        return p
    # every k-th element
    k = [int(rs.randint(1, 4)) for _ in shape]
    big = Pair.dense(cl, oracle.uniform(seed, int(np.prod([s * q for s, q in zip(shape, k)]))).reshape(
        [s * q for s, q in zip(shape, k)]))
    p = big
    for d, q in enumerate(k):
        if q > 1:
            p = p.step(d, q)
        if p.view.sizes[d] != shape[d]:
            p = p.narrow(d, 0, shape[d])
    return p


OPS2 = [("cadd1", lambda a, b: a.dev.add(b.dev), lambda a, b: oracle.pointwise("cadd", a.view, a.view, b.view, 1.0)),
        ("cadd_v", lambda a, b: a.dev.add(0.375, b.dev), lambda a, b: oracle.pointwise("cadd", a.view, a.view, b.view, 0.375)),
        ("cmul", lambda a, b: a.dev.cmul(b.dev), lambda a, b: oracle.pointwise("cmul", a.view, a.view, b.view)),
        ("copy", lambda a, b: a.dev.copy(b.dev), lambda a, b: oracle.pointwise("copy", a.view, b.view)),
        ("map", lambda a, b: a.dev.map_on_gpu(b.dev, "x = 1000*x + y*10"), lambda a, b: oracle.pointwise("map_c2", a.view, b.view))]


@pytest.mark.parametrize("seed", range(40))
def test_random_same_shape_operands(cl, seed):
    rs = np.random.RandomState(1000 + seed)
    nd = int(rs.randint(1, 5))
    shape = tuple(int(rs.choice([1, 2, 3, 4, 5, 7, 8, 16, 17, 33, 64])) for _ in range(nd))
    if rs.rand() < 0.3:                                       # now and then a plane big enough for full tiles
        shape = shape[:-2] + (int(rs.choice([64, 96, 130])), int(rs.choice([64, 128, 260]))) if nd >= 2 else (int(rs.choice([4096, 5000])),)
    for name, dev_op, host_op in OPS2:
        a = _same_shape_view(rs, cl, shape, 3 * seed + 1)
        b = _same_shape_view(rs, cl, shape, 3 * seed + 2)
        b_before = b.host_storage.copy()
        dev_op(a, b)
        host_op(a, b)
        assert_bit_equal(a.device_storage(), a.host_storage, f"seed {seed} {name} shape {shape} a{a.view.strides} b{b.view.strides}")
        assert_bit_equal(b.device_storage(), b_before, f"seed {seed} {name}: input modified")
    # three operands
    a, b, c = (_same_shape_view(rs, cl, shape, 3 * seed + 10 + i) for i in range(3))
    a.dev.addcmul(0.5, b.dev, c.dev)
    oracle.pointwise("addcmul", a.view, b.view, c.view, 0.5)
    assert_bit_equal(a.device_storage(), a.host_storage, f"seed {seed} addcmul shape {shape}")
    a.dev.map2_on_gpu(b.dev, c.dev, "x = sqrt(1000*x*x + y*10 + z*z)")
    oracle.pointwise("map2_c1", a.view, b.view, c.view)
    assert_bit_equal(a.device_storage(), a.host_storage, f"seed {seed} map2 shape {shape}")


@pytest.mark.parametrize("seed", range(25))
def test_random_view_chains_with_equal_element_counts(cl, seed):
    """Operands of different shapes pair up in logical order (the generic kernel)."""
    rs = np.random.RandomState(5000 + seed)
    n_target = None
    for attempt in range(50):
        shape_a = tuple(int(rs.choice([2, 3, 4, 6, 8, 12])) for _ in range(int(rs.randint(1, 4))))
        a = _random_view(rs, Pair.dense(cl, oracle.uniform(seed + 1, int(np.prod(shape_a))).reshape(shape_a)))
        n_target = int(np.prod(a.view.sizes))
        if n_target >= 2:
            break
    # b: any shape with the same count, as a strided slice of a bigger 1-d storage reshaped
    k = int(rs.randint(1, 4))
    flat = Pair(cl, oracle.uniform(seed + 2, n_target * k + 5), int(rs.randint(0, 5)), (n_target,), (k,))
    for name, dev_op, host_op in OPS2[:4]:
        before = flat.host_storage.copy()
        dev_op(a, flat)
        host_op(a, flat)
        assert_bit_equal(a.device_storage(), a.host_storage, f"seed {seed} {name} a{a.view.sizes}/{a.view.strides} k{k}")
        assert_bit_equal(flat.device_storage(), before, "input modified")
    dev = flat.dev
    dev.copy(a.dev)                                           # and the other way round
    oracle.pointwise("copy", flat.view, a.view)
    assert_bit_equal(flat.device_storage(), flat.host_storage, f"seed {seed} copy into the flat view")


@pytest.mark.parametrize("seed", range(20))
def test_random_reductions_on_views(cl, seed):
    rs = np.random.RandomState(9000 + seed)
    shape = tuple(int(rs.choice([2, 3, 5, 8, 16, 31, 64, 100])) for _ in range(int(rs.randint(1, 4))))
    p = _random_view(rs, Pair.dense(cl, oracle.normal(seed + 50, int(np.prod(shape))).reshape(shape)))
    g = p.view.gather()
    want = oracle.sumall(p.view)
    assert abs(p.dev.sum() - want) <= 1e-5 * max(abs(want), 1e-3 * np.sqrt(g.size))
    assert p.dev.max() == oracle.maxall(p.view) and p.dev.min() == oracle.minall(p.view)
    for d in range(len(p.view.sizes)):
        got = p.dev.sum(d + 1).float()
        exact = g.astype(np.float64).sum(axis=d, keepdims=True)
        assert got.shape == exact.shape
        assert np.all(np.abs(got - exact) <= 1e-5 * np.maximum(np.abs(exact), 1e-3))
        for kind in ("max", "min"):
            wv, wi = oracle.reduce_dim(kind, p.view, d)
            gv, gi = getattr(p.dev, kind)(d + 1)
            assert_bit_equal(gv.float(), wv, f"seed {seed} {kind} dim {d + 1} of {p.view.sizes}/{p.view.strides}")
            assert np.array_equal(gi.long(), wi)
