"""Pins the CPU oracle (oracle/th_oracle.c) before anything is compared with it.

Each check is chosen so that a plausible slip -- a dropped term, operands
swapped, a wrong index, a transposed stride -- makes it fail: IEEE fp32
arithmetic redone by numpy, exactly rounded sums (math.fsum), brute-force
index walks, closed forms, and the vectors of the reference's own tests
(tests/golden/reference_vectors.json).
"""
import math

import numpy as np
import pytest

import oracle
from oracle import View

F = np.float32


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).reshape(-1).view(np.uint32)


# --------------------------------------------------------------- MT19937 ---
def test_mt19937_known_answers():
    # first outputs of the reference implementation (mt19937ar.c) for the default seed 5489
    assert list(oracle.mt_raw(5489, 3)) == [3499211612, 581869302, 3890346734]


def test_mt19937_matches_numpy_legacy_stream():
    for seed in (1, 7, 12345):
        rs = np.random.RandomState(seed)
        want = rs.randint(0, 2 ** 32, size=2000, dtype=np.uint64).astype(np.uint32)
        # RandomState.randint on the full 32-bit range consumes one raw word per draw
        got = oracle.mt_raw(seed, 2000)
        assert np.array_equal(got, want)


def test_uniform_and_normal_ranges():
    u = oracle.uniform(3, 200000, -1.0, 1.0)
    assert u.dtype == np.float32 and u.min() >= -1.0 and u.max() < 1.0
    assert abs(float(u.mean())) < 0.01 and abs(float(u.var()) - 1 / 3) < 0.01
    raw = oracle.mt_raw(3, 5)
    assert np.array_equal(u[:5], (raw.astype(np.float64) / 2 ** 32 * 2 - 1).astype(np.float32))
    g = oracle.normal(6, 200000, 0.0, 1.0)
    assert abs(float(g.mean())) < 0.01 and abs(float(g.std()) - 1) < 0.01
    assert np.all(np.isfinite(g))


# ------------------------------------------------------------- pointwise ---
def test_pointwise_reference_pairs(golden):
    c = np.array(golden["pointwise_pairs"]["c"], dtype=F)
    d = np.array(golden["pointwise_pairs"]["d"], dtype=F)
    for op, want in [("cadd", c + d), ("cmul", c * d), ("cdiv", c / d), ("csub", c - d)]:
        r = View.contiguous(c.copy())
        oracle.pointwise(op, r, r, View.contiguous(d), 1.0)
        assert np.array_equal(bits(r.storage), bits(want)), op


def test_pointwise_scalar_forms(golden):
    c = np.array(golden["scalar_ops"]["c"], dtype=F)
    v = F(golden["scalar_ops"]["value"])
    for op, want in [("add_s", c + v), ("mul_s", c * v), ("div_s", c / v), ("sub_s", c + (-v)),
                     ("mulrecip_s", c * (F(1) / v))]:
        r = View.contiguous(c.copy())
        oracle.pointwise(op, r, r, None, float(v))
        assert np.array_equal(bits(r.storage), bits(want)), op
    # dividing and multiplying by the reciprocal really are different roundings somewhere
    x = oracle.uniform(11, 4096)
    a, b = View.contiguous(x.copy()), View.contiguous(x.copy())
    oracle.pointwise("div_s", a, a, None, 3.4)
    oracle.pointwise("mulrecip_s", b, b, None, 3.4)
    assert np.array_equal(a.storage, x / F(3.4)) and not np.array_equal(a.storage, b.storage)


def test_cadd_rounds_product_then_sum():
    # a + v*b with two roundings; a fused multiply-add would differ on some inputs
    rng = np.random.RandomState(0)
    a = rng.uniform(-1, 1, 50000).astype(F)
    b = rng.uniform(-1, 1, 50000).astype(F)
    v = F(0.3)
    r = View.contiguous(a.copy())
    oracle.pointwise("cadd", r, r, View.contiguous(b), float(v))
    two_roundings = a + (v * b)
    fused = (a.astype(np.float64) + np.float64(v) * b.astype(np.float64)).astype(F)
    assert np.array_equal(bits(r.storage), bits(two_roundings))
    assert not np.array_equal(two_roundings, fused)  # the check can tell the two apart


def test_config_expressions_closed_form():
    x, y, z = (oracle.uniform(s, 10000) for s in (1, 2, 3))
    r = View.contiguous(x.copy())
    oracle.pointwise("map2_c1", r, View.contiguous(y), View.contiguous(z))
    with np.errstate(invalid="ignore"):
        want = np.sqrt(F(1000) * x * x + y * F(10) + z * z)
    assert np.array_equal(np.isnan(r.storage), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(bits(r.storage[ok]), bits(want[ok]))
    r = View.contiguous(x.copy())
    oracle.pointwise("map_c2", r, View.contiguous(y))
    assert np.array_equal(bits(r.storage), bits(F(1000) * x + y * F(10)))


def test_pointwise_walks_strided_views_in_logical_order():
    base = np.arange(4 * 6 * 5, dtype=F)
    a = View.contiguous(base.reshape(4, 6, 5).copy())
    t = a.transpose(0, 2)                      # sizes (5,6,4), strides (1,5,30)
    dst = View.contiguous(np.zeros((5, 6, 4), dtype=F))
    oracle.pointwise("copy", dst, t)
    assert np.array_equal(dst.storage.reshape(5, 6, 4), base.reshape(4, 6, 5).transpose(2, 1, 0))
    n = a.narrow(2, 1, 3)                      # offset 1
    assert np.array_equal(n.gather(), base.reshape(4, 6, 5)[:, :, 1:4])
    s = a.step(2, 2)
    assert np.array_equal(s.gather(), base.reshape(4, 6, 5)[:, :, ::2])
    # same element count, different shapes: pairing is by logical position
    flat = View.contiguous(np.zeros(5 * 6 * 4, dtype=F))
    oracle.pointwise("copy", flat, t)
    assert np.array_equal(flat.storage, base.reshape(4, 6, 5).transpose(2, 1, 0).reshape(-1))
    with pytest.raises(ValueError):
        oracle.pointwise("copy", View.contiguous(np.zeros(7, dtype=F)), t)


# ---------------------------------------------------------------- reduce ---
def test_sumall_is_double_accumulated():
    x = oracle.uniform(5, 300001, 0.0, 1.0)
    got = oracle.sumall(View.contiguous(x))
    exact = math.fsum(float(v) for v in x)
    assert abs(got - exact) < 1e-7 * exact
    # an fp32 accumulator would be far off at this length: the check notices
    f32 = F(0)
    for v in x[:100000]:
        f32 = F(f32 + v)
    assert abs(float(f32) - math.fsum(float(v) for v in x[:100000])) > 1e-3
    assert oracle.sumall(View.contiguous(np.ones(12345, dtype=F))) == 12345.0
    ar = np.arange(1, 2001, dtype=F)
    assert oracle.sumall(View.contiguous(ar)) == 2000 * 2001 / 2
    assert oracle.prodall(View.contiguous(np.array([1, 2, 3, 4, 0.5], dtype=F))) == 12.0


def test_reduce_reference_vectors(golden):
    g = golden["matrixwide"]
    C = np.array(g["C"], dtype=F)
    v = View.contiguous(C)
    assert oracle.maxall(v) == g["max"] and oracle.minall(v) == g["min"] and oracle.sumall(v) == g["sum"]
    assert np.array_equal(oracle.reduce_dim("sum", v, 0)[0], np.array(g["sum_dim1"], dtype=F))
    assert np.array_equal(oracle.reduce_dim("sum", v, 1)[0], np.array(g["sum_dim2"], dtype=F))
    for kind in ("max", "min"):
        for dim in (0, 1):
            vals, idx = oracle.reduce_dim(kind, v, dim)
            assert np.array_equal(vals, np.array(g[f"{kind}_dim{dim + 1}"], dtype=F))
            assert np.array_equal(idx, np.array(g[f"arg{kind}_dim{dim + 1}"], dtype=np.int64))


def test_reduce_dim_brute_force_on_views():
    rng = np.random.RandomState(1)
    base = rng.uniform(-1, 1, (7, 9, 5)).astype(F)
    a = View.contiguous(base)
    for view, ref in [(a, base), (a.transpose(0, 2), base.transpose(2, 1, 0)),
                      (a.narrow(1, 2, 4), base[:, 2:6, :]), (a.step(2, 2), base[:, :, ::2])]:
        for dim in range(3):
            s, _ = oracle.reduce_dim("sum", view, dim)
            want = ref.astype(np.float64).sum(axis=dim, keepdims=True).astype(F)
            assert np.array_equal(s, want)
            for kind, fn, arg in (("max", np.max, np.argmax), ("min", np.min, np.argmin)):
                vals, idx = oracle.reduce_dim(kind, view, dim)
                assert np.array_equal(vals, fn(ref, axis=dim, keepdims=True))
                assert np.array_equal(idx, np.expand_dims(arg(ref, axis=dim), dim) + 1)


def test_max_min_ties_and_nan_rules():
    # ties keep the first position; the first NaN wins and stops the scan
    row = np.array([[1, 5, 5, 2, 5], [3, 3, 3, 3, 3]], dtype=F)
    vals, idx = oracle.reduce_dim("max", View.contiguous(row), 1)
    assert idx.ravel().tolist() == [2, 1]
    vals, idx = oracle.reduce_dim("min", View.contiguous(row), 1)
    assert idx.ravel().tolist() == [1, 1]
    nanrow = np.array([[1, np.nan, 7, np.nan, 9]], dtype=F)
    for kind in ("max", "min"):
        vals, idx = oracle.reduce_dim(kind, View.contiguous(nanrow), 1)
        assert np.isnan(vals[0, 0]) and idx[0, 0] == 2
    assert np.isnan(oracle.maxall(View.contiguous(nanrow))) and np.isnan(oracle.minall(View.contiguous(nanrow)))
    assert oracle.maxall(View.contiguous(np.array([-np.inf, -3, -np.inf], dtype=F))) == -3
    lead = np.array([[np.nan, 4, 5]], dtype=F)
    assert oracle.reduce_dim("max", View.contiguous(lead), 1)[1][0, 0] == 1


# ----------------------------------------------------------------- addmm ---
def test_addmm_reference_vector_and_numpy(golden):
    g = golden["blas_mm"]
    A, B = np.array(g["A"], dtype=F), np.array(g["B"], dtype=F)
    Z = np.zeros((2, 2), dtype=F)
    r = oracle.addmm_f64(0.0, View.contiguous(Z), 1.0, View.contiguous(A), View.contiguous(B))
    assert np.array_equal(r, np.array(g["expect"], dtype=np.float64))
    rng = np.random.RandomState(2)
    A = rng.normal(size=(37, 53)).astype(F)
    B = rng.normal(size=(53, 29)).astype(F)
    C = rng.normal(size=(37, 29)).astype(F)
    want = 0.5 * C.astype(np.float64) + 1.5 * (A.astype(np.float64) @ B.astype(np.float64))
    got = oracle.addmm_f64(0.5, View.contiguous(C), 1.5, View.contiguous(A), View.contiguous(B))
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    # asymmetric operands: a transposed or swapped product would not match
    assert not np.allclose(got, 0.5 * C + 1.5 * (B.T.astype(np.float64) @ A.T.astype(np.float64)).T[:, ::-1])
    # strided operands: A given as the transpose of a dense (K x M) array
    At = np.ascontiguousarray(A.T)
    got_t = oracle.addmm_f64(0.5, View.contiguous(C), 1.5, View.contiguous(At).transpose(0, 1), View.contiguous(B))
    assert np.array_equal(got_t, got)
    rows, cols = np.array([0, 5, 36]), np.array([28, 3, 0])
    samp = oracle.addmm_f64_sampled(rows, cols, 0.5, View.contiguous(C), 1.5, View.contiguous(A), View.contiguous(B))
    assert np.allclose(samp, want[rows, cols], rtol=1e-12)


# ---------------------------------------------------------------- layout ---
def _offsets(sizes, strides):
    idx = np.indices(sizes).reshape(len(sizes), -1)
    return (idx * np.array(strides).reshape(-1, 1)).sum(axis=0)


def test_collapse_preserves_every_offset():
    rng = np.random.RandomState(3)
    for _ in range(300):
        nd = rng.randint(1, 6)
        sizes = [int(rng.choice([1, 1, 2, 3, 4, 5])) for _ in range(nd)]
        # start dense, then perturb: transpose, widen a stride, or keep
        strides, z = [0] * nd, 1
        for d in reversed(range(nd)):
            strides[d] = z
            z *= sizes[d] * int(rng.choice([1, 1, 1, 2]))
        if nd > 1 and rng.rand() < 0.4:
            i, j = rng.choice(nd, 2, replace=False)
            sizes[i], sizes[j] = sizes[j], sizes[i]
            strides[i], strides[j] = strides[j], strides[i]
        csz, cst = oracle.collapse(sizes, strides)
        assert np.array_equal(_offsets(sizes, strides), _offsets(csz, cst))
        assert all(s > 1 for s in csz) or csz == [1]
        assert oracle.is_contiguous(sizes, strides) == (len(csz) == 1 and cst[0] == 1) or csz == [1]


def test_collapse_worked_layouts_of_the_strided_config():
    # 512x512x256 dense; transpose(0,2), stride-2 and narrow views
    assert oracle.collapse([256, 512, 512], [1, 256, 131072]) == ([256, 512, 512], [1, 256, 131072])
    assert oracle.collapse([512, 512, 128], [131072, 256, 2]) == ([2 ** 25], [2])
    assert oracle.collapse([512, 512, 128], [131072, 256, 1]) == ([262144, 128], [256, 1])
    assert oracle.collapse([512, 512, 256], [131072, 256, 1]) == ([2 ** 26], [1])
    # reduce dim is treated as size 1
    assert oracle.collapse([4096, 16384], [16384, 1], reduce_dim=0) == ([16384], [1])
    assert oracle.collapse([4096, 16384], [16384, 1], reduce_dim=1) == ([4096], [16384])
    assert oracle.collapse([1, 1], [1, 1]) == ([1], [1])


def test_overlap_rule():
    assert not oracle.overlapping([4, 5], [5, 1])
    assert not oracle.overlapping([5, 4], [1, 5])          # transposed: no overlap
    assert not oracle.overlapping([4, 5], [10, 2])         # holes
    assert oracle.overlapping([4, 5], [0, 1])              # expanded
    assert oracle.overlapping([4, 5], [3, 1])              # rows overlap
    assert oracle.overlapping([3, 4], [1, 1])              # unfold-like
    assert not oracle.overlapping([1, 1], [0, 0])
    rng = np.random.RandomState(4)
    for _ in range(200):
        nd = rng.randint(1, 4)
        sizes = [int(rng.randint(1, 5)) for _ in range(nd)]
        strides = [int(rng.randint(0, 7)) for _ in range(nd)]
        offs = _offsets(sizes, strides)
        brute = len(set(offs.tolist())) != len(offs)
        if oracle.overlapping(sizes, strides) != brute:
            # the rule is conservative: it may report overlap for interleaved but disjoint views
            assert oracle.overlapping(sizes, strides) and not brute


# ------------------------------------------------------ operator catalogue pins ---
def test_catalogue_special_values_and_identities():
    from oracle import catalogue as cat
    halves = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.49999997, -0.49999997, 2.4, -2.6, 8388609.0], dtype=np.float32)
    assert cat.unary("round", halves).tolist() == [1, 2, 3, -1, -2, -3, 0, -0.0, 2, -3, 8388609.0]
    assert cat.unary("sign", [-3.5, -0.0, 0.0, 7.0]).tolist() == [-1, 0, 0, 1]
    assert np.isnan(cat.unary("sign", [np.nan])[0]) == False and cat.unary("sign", [np.nan])[0] == 0   # both tests false
    assert cat.pown([2.0, -3.0, 0.5], 3).tolist() == [8.0, -27.0, 0.125]
    assert cat.pown([2.0, 4.0], -2).tolist() == [0.25, 0.0625]
    assert cat.pown([5.0], 0).tolist() == [1.0]
    assert cat.pow_value([2.0, 3.0], 2.0).tolist() == [4.0, 9.0]            # integer-valued exponent: exact
    assert abs(cat.pow_value([2.0], 0.5)[0] - np.float32(np.sqrt(2.0))) <= np.spacing(np.float32(1.4142135))
    assert cat.tpow(2.0, [0.0, 1.0, 10.0]).tolist() == [1.0, 2.0, 1024.0]
    assert cat.cpow([2.0, 9.0], [3.0, 0.5]).tolist() == [8.0, 3.0]
    assert cat.clamp([-2.0, 0.25, 9.0, np.nan], -1.0, 1.0).tolist() == [-1.0, 0.25, 1.0, 1.0]   # fmin(NaN, hi) = hi, then fmax(hi, lo) = hi
    assert cat.cmax([1.0, 5.0, -0.0], [2.0, 4.0, 0.0]).tolist() == [2.0, 5.0, -0.0]
    assert cat.cmin([1.0, 5.0], [2.0, 4.0]).tolist() == [1.0, 4.0]
    assert cat.cmax([1.0, 5.0], 3.0).tolist() == [3.0, 5.0]
    a, b = np.array([1.0, 2.0, 3.0, np.nan], dtype=np.float32), np.array([2.0, 2.0, 2.0, 2.0], dtype=np.float32)
    assert cat.compare("lt", a, b).tolist() == [1, 0, 0, 0] and cat.compare("ge", a, b).tolist() == [0, 1, 1, 0]
    assert cat.compare("eq", a, b).tolist() == [0, 1, 0, 0] and cat.compare("ne", a, b).tolist() == [1, 0, 1, 1]
    assert cat.compare("le", a, 2.0).tolist() == [1, 1, 0, 0] and cat.compare("gt", a, 2.0).tolist() == [0, 0, 1, 0]
    assert cat.masked_fill([1.0, 2.0, 3.0], [0.0, 1.0, -2.0], 9.0).tolist() == [1.0, 9.0, 9.0]
    # identities that a swapped argument or a wrong function breaks
    x = np.linspace(-0.9, 0.9, 101).astype(np.float32)
    assert np.allclose(cat.unary("sin", x) ** 2 + cat.unary("cos", x) ** 2, 1.0, atol=1e-6)
    assert np.allclose(cat.unary("cosh", x) ** 2 - cat.unary("sinh", x) ** 2, 1.0, atol=1e-5)
    assert np.allclose(cat.unary("sin", cat.unary("asin", x)), x, atol=1e-6)
    assert np.allclose(cat.unary("cos", cat.unary("acos", x)), x, atol=1e-6)
    assert np.allclose(cat.unary("tan", cat.unary("atan", x)), x, atol=1e-6)
    assert np.allclose(cat.unary("log1p", x), np.log(1.0 + x.astype(np.float64)), atol=1e-6)
    assert cat.atan2([1.0, -1.0, 0.0], [0.0, 0.0, -1.0]).tolist() == [np.float32(np.pi / 2), np.float32(-np.pi / 2), np.float32(np.pi)]


def test_catalogue_remaining_unary_names_by_special_values():
    """exp, log, tanh, floor, ceil, sqrt and abs: each name pinned by values that a swapped table entry (floor for
    ceil, exp for log, abs for sqrt ...) gets wrong."""
    from oracle import catalogue as cat
    bits = lambda a: np.asarray(a, dtype=np.float32).view(np.uint32).tolist()
    assert bits(cat.unary("floor", [-0.5, 0.5, -2.0, 2.75, -2.75])) == bits([-1.0, 0.0, -2.0, 2.0, -3.0])
    assert bits(cat.unary("ceil", [-0.5, 0.5, -2.0, 2.75, -2.75])) == bits([-0.0, 1.0, -2.0, 3.0, -2.0])    # ceil(-0.5) keeps the sign
    assert cat.unary("sqrt", [2.25, 0.0, 16.0, 1e-38]).tolist()[:3] == [1.5, 0.0, 4.0]
    assert np.isnan(cat.unary("sqrt", [-1.0])[0]) and bits(cat.unary("sqrt", [-0.0])) == bits([-0.0])
    assert bits(cat.unary("abs", [-0.0, -3.5, 3.5, -np.inf])) == bits([0.0, 3.5, 3.5, np.inf])              # sign bit cleared, also on zero
    assert cat.unary("exp", [0.0])[0] == 1.0 and cat.unary("log", [1.0])[0] == 0.0
    assert abs(float(cat.unary("exp", [1.0])[0]) - np.e) <= 3e-7 and abs(cat.unary("log", [np.float32(np.e)])[0] - 1.0) <= 1e-7   # one ulp
    assert cat.unary("exp", [-np.inf])[0] == 0.0 and cat.unary("log", [0.0])[0] == -np.inf and np.isnan(cat.unary("log", [-1.0])[0])
    x = np.linspace(-6.0, 6.0, 241).astype(np.float32)
    t = cat.unary("tanh", x)
    assert np.array_equal(t, -cat.unary("tanh", -x)) and np.all(np.abs(t) < 1.0) and t[120] == 0.0           # odd, bounded
    assert np.all(np.diff(t.astype(np.float64)) >= 0) and abs(t[-1] - 1.0) < 2e-5
    assert np.allclose(t, np.sinh(x.astype(np.float64)) / np.cosh(x.astype(np.float64)), atol=1e-6)
    # exp and log undo one another, sqrt undoes squaring, floor <= x <= ceil with a gap of 0 or 1
    y = np.linspace(0.05, 20.0, 400).astype(np.float32)
    assert np.allclose(cat.unary("log", cat.unary("exp", y)), y, rtol=2e-6)
    assert np.allclose(cat.unary("sqrt", (y * y).astype(np.float32)), y, rtol=1e-6)
    f, c = cat.unary("floor", x), cat.unary("ceil", x)
    assert np.all(f <= x) and np.all(x <= c) and set((c - f).tolist()) <= {0.0, 1.0}


def test_scan_norm_truth_closed_forms():
    from oracle import catalogue as cat
    n = 3000
    assert np.array_equal(cat.cumulate(np.ones(n, dtype=np.float32), 0), np.arange(1, n + 1, dtype=np.float32))
    k = np.arange(1, n + 1, dtype=np.float64)
    assert np.array_equal(cat.cumulate(np.arange(1, n + 1, dtype=np.float32), 0), (k * (k + 1) / 2).astype(np.float32))
    assert np.array_equal(cat.cumulate(np.full(30, 2.0, dtype=np.float32), 0, prod=True), (2.0 ** np.arange(1, 31)).astype(np.float32))
    # a python loop with an fp64 running value on a small 2-d case, both axes
    x = oracle.uniform(3, 6 * 7).reshape(6, 7)
    for axis in (0, 1):
        want = np.empty_like(x)
        for line in range(x.shape[1 - axis]):
            acc = 0.0
            for r in range(x.shape[axis]):
                idx = (r, line) if axis == 0 else (line, r)
                acc += float(x[idx])
                want[idx] = np.float32(acc)
        assert np.array_equal(cat.cumulate(x, axis), want)
    # fp64 running value matters: 2^24 + 1 + 1 ... stays exact in fp64, then rounds
    big = np.array([16777216.0, 1.0, 1.0, 1.0], dtype=np.float32)
    assert cat.cumulate(big, 0).tolist() == [16777216.0, 16777216.0, 16777218.0, 16777220.0]
    v = np.array([[3.0, -4.0, 0.0], [0.0, 0.0, -2.0]], dtype=np.float32)
    assert cat.norm(v, 2) == 29.0 ** 0.5 or abs(cat.norm(v, 2) - np.float32(29.0 ** 0.5)) < 1e-6
    assert cat.norm(v, 1) == 9.0 and cat.norm(v, 0) == 3.0
    assert cat.norm(v, 2, axis=1).ravel().tolist() == [5.0, 2.0] and cat.norm(v, 0, axis=0).ravel().tolist() == [1.0, 1.0, 1.0]
    assert cat.truth([0.0, 0.5, -0.99, 1.0, -1.0, 2.5]).tolist() == [False, False, False, True, True, True]


def test_level12_small_integer_cases(golden):
    from oracle import catalogue as cat
    # the reference's own test matrices (src/test/unit_tensor.lua:413-438): {{1,2,-1},{3,4,0}} . {{0,1},{1,2},{4,5}}
    A = np.array([[1, 2, -1], [3, 4, 0]], dtype=np.float32)
    B = np.array([[0, 1], [1, 2], [4, 5]], dtype=np.float32)
    assert cat.addmv(0.0, np.zeros(2), 1.0, A, B[:, 0]).tolist() == [-2.0, 4.0]      # first column of {{-2,0},{4,11}}
    assert cat.addmv(2.0, np.array([1.0, 1.0]), 1.0, A, B[:, 1]).tolist() == [2.0, 13.0]
    assert cat.dot([1, 2, 3], [4, -5, 6]) == 12.0
    assert cat.addr(1.0, np.ones((2, 3)), 2.0, [1, 2], [3, 4, 5]).tolist() == [[7, 9, 11], [13, 17, 21]]
    assert cat.addr(0.5, np.full((2, 2), 4.0), 1.0, [1, -1], [2, 3]).tolist() == [[4, 5], [0, -1]]


def test_indexed_movement_hand_cases():
    from oracle import catalogue as cat
    a = np.arange(1, 13, dtype=np.float32).reshape(3, 4)             # rows 1..4 / 5..8 / 9..12
    assert cat.index_select(a, 0, [3, 1, 1]).tolist() == [[9, 10, 11, 12], [1, 2, 3, 4], [1, 2, 3, 4]]
    assert cat.index_select(a, 1, [4, 2]).tolist() == [[4, 2], [8, 6], [12, 10]]
    z = np.zeros((3, 2), dtype=np.float32)
    s = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    assert cat.index_copy(z, 0, [2, 3, 2], s).tolist() == [[0, 0], [5, 6], [3, 4]]     # target 2 named twice: last wins
    assert cat.index_fill(a, 1, [1, 3], -1.0)[0].tolist() == [-1, 2, -1, 4]
    g = cat.gather(a, 1, np.array([[1, 1], [4, 2], [3, 3]]))
    assert g.tolist() == [[1, 1], [8, 6], [11, 11]]
    g0 = cat.gather(a, 0, np.array([[3, 2, 1, 1]]))
    assert g0.tolist() == [[9, 6, 3, 4]]
    sc = cat.scatter(np.zeros((3, 4), dtype=np.float32), 0, np.array([[3, 2, 1, 1]]), np.array([[7, 8, 9, 10]], dtype=np.float32))
    assert sc.tolist() == [[0, 0, 9, 10], [0, 8, 0, 0], [7, 0, 0, 0]]
    assert cat.scatter(np.zeros((2, 2), dtype=np.float32), 1, np.array([[2], [1]]), 5.0).tolist() == [[0, 5], [5, 0]]
    # gather undoes scatter at the scattered positions
    idx = np.array([[2, 3, 1, 2], [1, 1, 3, 3]])
    vals = np.array([[1, 2, 3, 4], [5, 6, 7, 8]], dtype=np.float32)
    assert np.array_equal(cat.gather(cat.scatter(np.zeros((3, 4), dtype=np.float32), 0, idx, vals), 0, idx), vals)
    m = np.array([[0, 1, 0, 2], [1, 0, 0, 0], [0, 0, -1, 0]], dtype=np.float32)
    assert cat.masked_select(a, m).tolist() == [2, 4, 5, 11]
    assert cat.masked_copy(a, m, [-1, -2, -3, -4, -5])[0].tolist() == [1, -1, 3, -2]
    assert cat.masked_copy(a, m, [-1, -2, -3, -4])[2].tolist() == [9, 10, -4, 12]


# ------------------------------------------- expression evaluator (expr_host) ---
# oracle/expr_host.py judges every apply/map/map2 string other than the two
# configuration strings, so its text rewrite and its arithmetic are pinned here:
# the rewrite against the substitutions the reference makes
# (src/lib/THClTensorMathPointwise.cpp:79-146) on the strings of its own tests
# (src/test/unit_tensor.lua:583-635), the arithmetic against IEEE fp32 operations
# written out one rounding at a time with numpy.
def test_expr_rewrite_reference_strings():
    from oracle import expr_host as eh
    # the pointer syntax passes through untouched, the x/y/z syntax turns into it
    raw1 = "*out = sqrt(*out + 3) + exp(*out)"
    raw2 = "*out = sqrt(*out * *out + *in1 * *in1 + 3 + exp(*in1))"
    raw3 = "*out = sqrt(*out * *out + *in1 * *in1 + *in2 + 3 + exp(*in2))"
    assert eh.rewrite(raw1, 1) == raw1 and eh.rewrite(raw2, 2) == raw2 and eh.rewrite(raw3, 3) == raw3
    assert eh.rewrite("x = sqrt(x + 3) + exp(x)", 1) == "(*out) = sqrt((*out) + 3) + exp((*out))"
    assert eh.rewrite("x = sqrt(x * x + y * y + 3 + exp(y))", 2) == \
        "(*out) = sqrt((*out) * (*out) + (*in1) * (*in1) + 3 + exp((*in1)))"
    assert eh.rewrite("x = sqrt(x * x + y * y + z + 3 + exp(z))", 3) == \
        "(*out) = sqrt((*out) * (*out) + (*in1) * (*in1) + (*in2) + 3 + exp((*in2)))"
    # a call with fewer tensors leaves the later letters alone (apply replaces x only, map x and y)
    assert eh.rewrite("x = y + z", 1) == "(*out) = y + z"
    assert eh.rewrite("x = y + z", 2) == "(*out) = (*in1) + z"
    # names that merely contain x, y or z are not variables
    assert eh.rewrite("x = max(x, y) + hypot(x, y) + copysign(x, z) + exp(y)", 3) == \
        "(*out) = max((*out), (*in1)) + hypot((*out), (*in1)) + copysign((*out), (*in2)) + exp((*in1))"
    assert eh.rewrite("x = xx + y_1 + zeta", 3) == "(*out) = xx + y_1 + zeta"


def test_expr_rewrite_literals():
    from oracle import expr_host as eh
    assert eh.rewrite("x = 1000*x + 0.5 + 1e-3 + 2. + .25 + 3.5f + 7", 1) == \
        "(*out) = 1000*(*out) + 0.5f + 1e-3f + 2.f + .25f + 3.5f + 7"
    assert eh.rewrite("x = 1.5e+2*x - 10/4", 1) == "(*out) = 1.5e+2f*(*out) - 10/4"
    assert eh.rewrite("x = y2 + 3.25F", 1) == "(*out) = y2 + 3.25F"


def _ulps(a, b):
    """Distance in units of the last place between two finite fp32 arrays."""
    def key(v):
        i = np.ascontiguousarray(v, dtype=F).view(np.int32).astype(np.int64)
        return np.where(i < 0, -(i & 0x7FFFFFFF), i)
    return np.abs(key(a) - key(b))


def test_expr_evaluate_exact_strings_are_ieee_fp32():
    from oracle import expr_host as eh
    n = 4096
    x, y, z = (oracle.uniform(40 + i, n, -0.5, 0.5) for i in range(3))
    k1000, k10, half, milli, quarter, two = F(1000), F(10), F(0.5), F(1e-3), F(0.25), F(2)

    # 1000*x*x + y*10 + z*z associates left to right: ((1000*x)*x + y*10) + z*z, then one correctly rounded sqrt
    with np.errstate(invalid="ignore"):
        want = np.sqrt(((k1000 * x) * x + y * k10) + z * z)
    assert want.dtype == F
    assert np.array_equal(bits(eh.evaluate("x = sqrt(1000*x*x + y*10 + z*z)", x, y, z)), bits(want))

    # two roundings, not one: the fused form differs on some elements and must not be what the evaluator gives
    two_roundings = k1000 * x + y * k10
    fused = (k1000.astype(np.float64) * x.astype(np.float64) + (y * k10).astype(np.float64)).astype(F)
    assert np.any(bits(two_roundings) != bits(fused)), "inputs do not separate fused from unfused"
    got = eh.evaluate("x = 1000*x + y*10", x, y)
    assert np.array_equal(bits(got), bits(two_roundings))
    assert np.array_equal(bits(eh.evaluate("*out = 1000 * *out + *in1 * 10", x, y)), bits(two_roundings))

    # literals are fp32: 1e-3 as a double would round differently
    want = x * half + milli
    as_double = (x.astype(np.float64) * 0.5 + 1e-3).astype(F)
    assert np.any(bits(want) != bits(as_double))
    assert np.array_equal(bits(eh.evaluate("x = x * 0.5 + 1e-3", x)), bits(want))

    assert np.array_equal(bits(eh.evaluate("x = (x > 0.25) ? x : 2*x", x)), bits(np.where(x > quarter, x, two * x)))
    assert np.array_equal(bits(eh.evaluate("x = max(x, y) - min(x, y)", x, y)), bits(np.maximum(x, y) - np.minimum(x, y)))
    # strings the GPU tests use on views
    assert np.array_equal(bits(eh.evaluate("x = x*y + z", x, y, z)), bits(x * y + z))
    assert np.array_equal(bits(eh.evaluate("x = x + 2*y - z", x, y, z)), bits((x + two * y) - z))
    assert np.array_equal(bits(eh.evaluate("x = x*y + x", x, y)), bits(x * y + x))
    assert np.array_equal(bits(eh.evaluate("x = x - y", x, y)), bits(x - y))


def test_expr_evaluate_operand_binding():
    from oracle import expr_host as eh
    x = np.array([1.0, 2.0, 3.0], dtype=F)
    y = np.array([10.0, 20.0, 30.0], dtype=F)
    z = np.array([100.0, 200.0, 300.0], dtype=F)
    # x is the tensor written, y the first source, z the second: an exchange of any two changes the answer
    assert eh.evaluate("x = x + 2*y + 4*z", x, y, z).tolist() == [421.0, 842.0, 1263.0]
    assert eh.evaluate("*out = *out + 2 * *in1 + 4 * *in2", x, y, z).tolist() == [421.0, 842.0, 1263.0]
    assert eh.evaluate("x = y - x", x, y).tolist() == [9.0, 18.0, 27.0]
    assert eh.evaluate("x = z", x, y, z).tolist() == [100.0, 200.0, 300.0]
    # the inputs are left alone; only the returned array carries the result
    assert x.tolist() == [1.0, 2.0, 3.0] and y.tolist() == [10.0, 20.0, 30.0]
    # a statement may read the old x after naming it on the left
    assert eh.evaluate("x = x * x", np.array([3.0, -4.0], dtype=F)).tolist() == [9.0, 16.0]
    # integer literals promote to float as OpenCL C does: 10/4 stays an integer division, 10/4.0 does not
    assert eh.evaluate("x = x + 10/4", np.zeros(1, dtype=F)).tolist() == [2.0]
    assert eh.evaluate("x = x + 10/4.0", np.zeros(1, dtype=F)).tolist() == [2.5]


def test_expr_evaluate_prelude_functions():
    from oracle import expr_host as eh
    v = np.array([-2.5, -0.0, 0.0, 0.75, 3.0], dtype=F)
    assert eh.evaluate("x = sign(x)", v).tolist() == [-1.0, 0.0, 0.0, 1.0, 1.0]
    assert eh.evaluate("x = clamp(x, -1.0, 1.0)", v).tolist() == [-1.0, -0.0, 0.0, 0.75, 1.0]
    assert eh.evaluate("x = pown(x, 3)", v).tolist() == [-15.625, -0.0, 0.0, 0.421875, 27.0]
    assert eh.evaluate("x = fabs(x) + floor(x) + ceil(x)", v).tolist() == [-2.5, 0.0, 0.0, 1.75, 9.0]
    assert eh.evaluate("x = max(x, 1.0) + min(x, -1.0)", v).tolist() == [-1.5, 0.0, 0.0, 0.0, 2.0]


def test_expr_evaluate_transcendental_strings_within_one_ulp():
    from oracle import expr_host as eh
    n = 3000
    x, y, z = (oracle.uniform(50 + i, n, -0.5, 0.5) for i in range(3))
    three = F(3)
    e32 = lambda v: np.exp(v.astype(np.float64)).astype(F)       # exp in fp64, rounded once
    # the function itself: within one unit of the correctly rounded value
    assert _ulps(eh.evaluate("x = exp(x)", x), e32(x)).max() <= 1
    # (the host C library documents 2 units for tanhf, 1 for the others)
    for fn, ref, bound in (("log", np.log, 1), ("sin", np.sin, 1), ("cos", np.cos, 1), ("tanh", np.tanh, 2)):
        arg = x + F(1.0)
        assert _ulps(eh.evaluate(f"x = {fn}(x)", arg), ref(arg.astype(np.float64)).astype(F)).max() <= bound, fn
    assert _ulps(eh.evaluate("x = pow(x, y)", x + F(1.0), y), np.power((x + F(1.0)).astype(np.float64), y.astype(np.float64)).astype(F)).max() <= 1
    # the reference's three test statements, both spellings: fp32 steps with the exponential rounded from fp64.
    # One unit of error in exp(.) (about 1) moves the sum under the root (about 4) by at most one of its units,
    # and the root halves relative errors, so the result stays within one unit.
    cases = [
        ("x = sqrt(x + 3) + exp(x)", "*out = sqrt(*out + 3) + exp(*out)", (x,),
         np.sqrt(x + three) + e32(x), np.sqrt(x.astype(np.float64) + 3) + np.exp(x.astype(np.float64))),
        ("x = sqrt(x * x + y * y + 3 + exp(y))", "*out = sqrt(*out * *out + *in1 * *in1 + 3 + exp(*in1))", (x, y),
         np.sqrt(((x * x + y * y) + three) + e32(y)),
         np.sqrt(x.astype(np.float64) ** 2 + y.astype(np.float64) ** 2 + 3 + np.exp(y.astype(np.float64)))),
        ("x = sqrt(x * x + y * y + z + 3 + exp(z))", "*out = sqrt(*out * *out + *in1 * *in1 + *in2 + 3 + exp(*in2))", (x, y, z),
         np.sqrt((((x * x + y * y) + z) + three) + e32(z)),
         np.sqrt(x.astype(np.float64) ** 2 + y.astype(np.float64) ** 2 + z.astype(np.float64) + 3 + np.exp(z.astype(np.float64)))),
    ]
    for xyz, raw, arrs, stepwise, exact64 in cases:
        a = eh.evaluate(xyz, *arrs)
        b = eh.evaluate(raw, *arrs)
        assert np.array_equal(bits(a), bits(b)), xyz                    # the two spellings are one statement
        assert stepwise.dtype == F
        assert _ulps(a, stepwise).max() <= 1, xyz
        assert _ulps(a, exact64.astype(F)).max() <= 2, xyz               # and close to the fp64 value of the whole statement
