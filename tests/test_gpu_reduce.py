"""GPU parity: reduce-all (host scalar and point tensor), reduce along a
dimension, max/min with positions -- against the CPU oracle, through the C ABI.
Sums: 1e-5 relative (the device accumulates in fp64 like Torch7's CPU path, so
they are in practice equal or one ulp apart); max/min values and all positions:
exact.  Cases follow src/test/unit_tensor.lua:488-496,637-657,735-832."""
import numpy as np
import pytest

import oracle
from oracle import View
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32
SUM_RTOL = 1e-5


def close_sum(got, want64):
    want = np.asarray(want64, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    assert np.all(np.abs(got - want) <= SUM_RTOL * np.abs(want) + 1e-30), (got, want)
    # much tighter in practice: fp64 accumulation leaves at most the final rounding
    assert np.all(np.abs(got - want) <= 1.5 * np.spacing(np.abs(want).astype(F)).astype(np.float64))


def test_reference_matrix(cl, golden):
    g = golden["matrixwide"]
    C = cl.ClTensor(g["C"])
    assert C.max() == g["max"] and C.min() == g["min"] and C.sum() == g["sum"]
    assert C.sum(1).float().tolist() == g["sum_dim1"] and C.sum(2).float().tolist() == g["sum_dim2"]
    for kind in ("max", "min"):
        for dim in (1, 2):
            vals, idx = getattr(C, kind)(dim)
            assert vals.float().tolist() == g[f"{kind}_dim{dim}"]
            assert idx.long().tolist() == g[f"arg{kind}_dim{dim}"]
            vals2, idx2 = getattr(C, f"{kind}_long")(dim)
            assert idx2.tolist() == g[f"arg{kind}_dim{dim}"] and idx2.dtype == np.int64


@pytest.mark.parametrize("n", [1, 2, 3, 5, 63, 64, 65, 1023, 1024, 1025, 4099, 65537, 1 << 20, (1 << 22) + 7])
def test_reduce_all_lengths(cl, n):
    x = oracle.uniform(5, n, -0.5, 0.5)
    X, v = cl.ClTensor(x), View.contiguous(x)
    close_sum(X.sum(), oracle.sumall(v))
    assert X.max() == oracle.maxall(v) and X.min() == oracle.minall(v)
    pt = cl.ClTensor()
    pt.sum(X)
    assert pt.nDimension() == 0 and pt.nElement() == 0
    close_sum(pt.s(), oracle.sumall(v))
    pt.max(X)
    assert pt.s() == oracle.maxall(v)
    pt.min(X)
    assert pt.s() == oracle.minall(v)


def test_reduce_all_reference_sizes(cl, golden):
    # the two shapes of test_reduceAll, with the reference's (loose) bounds and ours
    t = golden["tolerances"]
    for shape, bound in ((t["reduceall_two_pass_shape"], t["reduceall_two_pass_abs"]),
                         (t["reduceall_one_pass_shape"], t["reduceall_one_pass_abs"])):
        n = int(np.prod(shape))
        x = oracle.uniform(9, n, -0.5, 0.5)
        got = cl.ClTensor(x.reshape(shape)).sum()
        want = oracle.sumall(View.contiguous(x))
        assert abs(got - want) < bound
        close_sum(got, want)


def test_reduce_all_closed_forms_and_determinism(cl):
    assert cl.ClTensor(np.ones(1 << 21, dtype=F)).sum() == float(1 << 21)
    ar = np.arange(1, 4097, dtype=F)
    assert cl.ClTensor(ar).sum() == 4096 * 4097 / 2
    assert cl.ClTensor(np.array([1, 2, 3, 4, 0.5], dtype=F)).prod() == 12.0
    x = oracle.uniform(13, (1 << 21) + 3)
    X = cl.ClTensor(x)
    first = X.sum()
    assert all(X.sum() == first for _ in range(5))
    # linearity: doubling every element doubles the sum exactly (same combine order, exact scaling)
    assert cl.ClTensor(x).mul(2.0).sum() == 2 * first


def test_reduce_all_special_values(cl):
    x = oracle.uniform(14, 100000)
    x[777] = np.nan
    X = cl.ClTensor(x)
    assert np.isnan(X.sum()) and np.isnan(X.max()) and np.isnan(X.min())     # Torch7's CPU rule: NaN propagates
    y = np.full(5000, -np.inf, dtype=F)
    assert cl.ClTensor(y).max() == -np.inf
    y[4321] = -3.0
    assert cl.ClTensor(y).max() == -3.0 and cl.ClTensor(y).min() == -np.inf
    assert cl.ClTensor(np.array([-0.0, 0.0], dtype=F)).sum() == 0.0
    # a NaN anywhere in a stream of whole and ragged tiles (quiet or signalling), infinities among numbers
    for n in (1, 5, 1023, 4099, (1 << 20) + 7):
        a = oracle.uniform(15 + n, n)
        A = cl.ClTensor(a)
        assert A.max() == a.max() and A.min() == a.min()
        for pos in {0, n // 2, n - 1}:
            for bits in (0x7fc00000, 0x7f800001, 0xffc00000):
                b = a.copy()
                b.view(np.uint32)[pos] = bits
                B = cl.ClTensor(b)
                assert np.isnan(B.max()) and np.isnan(B.min()), (n, pos, hex(bits))
        if n >= 4:
            b = a.copy()
            b[n // 3], b[n // 2] = np.inf, -np.inf
            assert cl.ClTensor(b).max() == np.inf and cl.ClTensor(b).min() == -np.inf


def test_reduce_all_on_views_walked_in_units_of_four(cl):
    """Views whose innermost run is dense, a multiple of 4 long and 16-byte aligned in every row are walked four
    elements at a time; neighbours that miss one of the conditions take the one-element walk.  Both against the oracle."""
    base = oracle.uniform(16, 96 * 64 * 72).reshape(96, 64, 72)
    p = Pair.dense(cl, base)
    views = (p.narrow(2, 4, 32), p.narrow(2, 8, 64).narrow(1, 3, 40), p.narrow(0, 5, 80).narrow(2, 0, 36),     # aligned runs
             p.narrow(2, 3, 32), p.narrow(2, 4, 30), p.transpose(0, 1).narrow(2, 12, 48), p.step(1, 2).narrow(2, 16, 40))
    for q in views:
        close_sum(q.dev.sum(), oracle.sumall(q.view))
        assert q.dev.max() == oracle.maxall(q.view) and q.dev.min() == oracle.minall(q.view)
    big = oracle.uniform(17, 2048 * 4096).reshape(2048, 4096)
    b = Pair.dense(cl, big)
    for q in (b.narrow(1, 0, 2048), b.narrow(1, 4, 4088), b.step(0, 2)):
        close_sum(q.dev.sum(), oracle.sumall(q.view))
        assert q.dev.max() == oracle.maxall(q.view)
    x = big.copy()
    x[1000, 77] = np.nan
    assert np.isnan(Pair.dense(cl, x).narrow(1, 0, 2048).dev.max()) and not np.isnan(Pair.dense(cl, x).narrow(1, 2048, 2048).dev.max())


def test_scalars_handed_to_the_host_in_a_row(cl):
    """Scalar results reach the host through one pinned word pair with a tag per call: many calls in a row,
    of different kinds and sizes, must each return their own value (no stale one from the call before)."""
    sizes = (1, 7, 1000, 4097, 1 << 16, (1 << 20) + 3)
    tensors = [(n, cl.ClTensor(np.full(n, 1.0 + i, dtype=F))) for i, n in enumerate(sizes)]
    pt = cl.ClTensor()
    for rep in range(300):
        i = rep % len(tensors)
        n, t = tensors[i]
        v = 1.0 + i
        assert t.sum() == F(n) * F(v)
        assert t.max() == v and t.min() == v
        assert t.dot(t) == float(F(n * v * v))
        pt.sum(t)
        assert pt.s() == F(n) * F(v)
    big = cl.ClTensor(np.ones(1 << 26, dtype=F))              # a reduction long enough to outlast a short poll
    assert big.sum() == float(1 << 26) and tensors[0][1].sum() == 1.0 and big.sum() == float(1 << 26)


def test_reduce_all_on_views(cl):
    base = oracle.uniform(15, 40 * 30 * 20).reshape(40, 30, 20)
    p = Pair.dense(cl, base)
    for q in (p.transpose(0, 2), p.narrow(2, 3, 9), p.step(2, 2), p.narrow(0, 7, 1), p.transpose(0, 1).narrow(1, 2, 11)):
        close_sum(q.dev.sum(), oracle.sumall(q.view))
        assert q.dev.max() == oracle.maxall(q.view) and q.dev.min() == oracle.minall(q.view)
    mis = Pair(cl, base.reshape(-1), 3, (5001,), (1,))
    close_sum(mis.dev.sum(), oracle.sumall(mis.view))
    assert cl.ClTensor().sum() == 0.0            # empty tensor: the identity


def _check_dim(cl, pair, dim0):
    """All three reductions along 0-based dim of a Pair, values + positions."""
    dim = dim0 + 1
    want, _ = oracle.reduce_dim("sum", pair.view, dim0)
    got = pair.dev.sum(dim)
    assert got.size() == want.shape
    exact64 = pair.view.gather().astype(np.float64).sum(axis=dim0, keepdims=True)
    close_sum(got.float(), exact64)
    for kind in ("max", "min"):
        wv, wi = oracle.reduce_dim(kind, pair.view, dim0)
        gv, gi = getattr(pair.dev, kind)(dim)
        assert_bit_equal(gv.float(), wv, f"{kind} values dim {dim}")
        assert np.array_equal(gi.long(), wi), f"{kind} positions dim {dim}"
        gv2, gi2 = getattr(pair.dev, f"{kind}_long")(dim)
        assert np.array_equal(gi2, wi) and np.array_equal(gv2.float(), wv)


@pytest.mark.parametrize("shape", [(5, 2), (60, 50), (3, 2000), (2000, 3), (7, 128), (129, 64), (33, 4096), (4096, 33),
                                   (17, 9, 13), (4, 300, 8), (2, 3, 4, 5), (1, 77), (77, 1), (256, 2048),
                                   # few long slices (cut into pieces over blocks), slices of 1..16 elements (a thread each),
                                   # fewer than 64 column units (a wave's spare lanes take further rows)
                                   (1, 1 << 20), (3, 300001), (5, 1 << 18), (1 << 20, 1), (300000, 3), (1 << 18, 4), (70000, 16),
                                   (100000, 12), (40000, 40), (2, 50000, 8), (3, 20000, 5), (70000, 100), (20000, 252)])
def test_reduce_dim_shapes(cl, shape):
    x = oracle.normal(6, int(np.prod(shape))).reshape(shape)
    p = Pair.dense(cl, x)
    for d in range(len(shape)):
        _check_dim(cl, p, d)


def test_reduce_dim_on_views_like_the_reference_tests(cl):
    # A:t():sum(d), A:narrow(..):t():sum(d)  (src/test/unit_tensor.lua:759-775)
    x = oracle.uniform(16, 60 * 50, -0.5, 0.5).reshape(60, 50)
    p = Pair.dense(cl, x)
    for q in (p.transpose(0, 1), p.narrow(0, 9, 30).transpose(0, 1), p.narrow(1, 9, 30).transpose(0, 1),
              p.step(1, 2), p.narrow(1, 1, 33)):
        for d in (0, 1):
            _check_dim(cl, q, d)
    y = oracle.uniform(17, 12 * 10 * 16).reshape(12, 10, 16)
    p3 = Pair.dense(cl, y)
    for q in (p3.transpose(0, 2), p3.transpose(1, 2), p3.narrow(2, 4, 8), p3.step(0, 3)):
        for d in range(3):
            _check_dim(cl, q, d)


@pytest.mark.parametrize("rows,cols,pitch,first", [(300, 256, 259, 1), (300, 256, 260, 0), (257, 1024, 1027, 2), (64, 4100, 4101, 1),
                                                   (2000, 64, 67, 3), (40, 20000, 20003, 1), (5000, 8, 11, 1)])
def test_reduce_dim_on_rows_that_start_at_odd_elements(cl, rows, cols, pitch, first):
    """A block cut out of a wider matrix: a multiple of 4 columns, but rows that start at element offsets which are no
    multiple of 4, so the units of four are read with 16-byte loads that need no alignment.  Both dims, values and
    positions, against the oracle."""
    x = oracle.normal(19, rows * pitch).reshape(rows, pitch)
    p = Pair.dense(cl, x).narrow(1, first, cols)
    for d in (0, 1):
        _check_dim(cl, p, d)
    assert_bit_equal(np.float32(p.dev.max()), np.float32(p.view.gather().max()))
    got, want = p.dev.sum(), float(p.view.gather().astype(np.float64).sum())
    assert abs(got - want) <= 1e-5 * abs(want) + 1e-3


@pytest.mark.parametrize("shape", [(300, 9), (300, 13), (5000, 8191 // 7), (64, 4099), (2049, 255), (31, 70001), (20, 11), (40000, 10)])
def test_reduce_dim_over_widths_that_are_no_multiple_of_four(cl, shape):
    """Along dim 1 of a matrix whose width is no multiple of 4 the units of four columns still apply: the last unit is
    moved back to end with the row and repeats up to three columns, bit for bit.  Values and positions, planted
    ties in the repeated columns included."""
    x = oracle.normal(23, int(np.prod(shape))).reshape(shape)
    x[3, -2] = x[1, -2] = x[:, -2].max() + 1.0          # a tie in a column that two units cover
    x[2, -1] = x[0, -1] = x[:, -1].min() - 1.0
    p = Pair.dense(cl, x)
    for d in (0, 1):
        _check_dim(cl, p, d)
    _check_dim(cl, p.narrow(1, 1, shape[1] - 2), 0)     # the same inside a wider matrix


@pytest.mark.parametrize("shape", [(40, 65), (300, 131), (33, 4099), (7, 70001), (2, 300003), (5000, 67), (64, 1023), (3, 8191)])
def test_reduce_dim_over_slices_whose_length_is_no_multiple_of_four(cl, shape):
    """Along the dense dim, slices of 64 elements or more are walked in units of four whatever their length; the last
    one to three elements are taken singly.  Extremes planted in those last elements and ties between them and the
    units; long slices are cut over blocks."""
    x = oracle.normal(29, int(np.prod(shape))).reshape(shape)
    x[0, -1] = x[0].max() + 1.0                       # the maximum is the very last element
    x[1, -2] = x[1, 3] = x[1].min() - 1.0             # a tie between a unit and the tail: the first position wins
    if shape[0] > 2:
        x[2, :] = x[2, 0]                             # every element equal: position 1
    p = Pair.dense(cl, x)
    _check_dim(cl, p, 1)
    _check_dim(cl, p.narrow(1, 1, shape[1] - 1), 1)   # slices that start at odd elements of a wider matrix


def test_positions_ties_and_nans(cl):
    row = np.array([[1, 5, 5, 2, 5], [3, 3, 3, 3, 3]], dtype=F)
    R = cl.ClTensor(row)
    assert R.max(2)[1].long().ravel().tolist() == [2, 1]
    assert R.min(2)[1].long().ravel().tolist() == [1, 1]
    assert R.max(1)[1].long().ravel().tolist() == [2, 1, 1, 2, 1]
    # long constant rows: every tree shape must still report position 1
    for n in (64, 257, 5000):
        c = cl.ClTensor(np.full((3, n), F(2.5)))
        assert c.max(2)[1].long().ravel().tolist() == [1, 1, 1] and c.min(2)[1].long().ravel().tolist() == [1, 1, 1]
        ct = cl.ClTensor(np.full((n, 3), F(2.5)))
        assert ct.max(1)[1].long().ravel().tolist() == [1, 1, 1]
    # planted ties far apart, and NaNs: first NaN wins (Torch7's CPU rule)
    x = oracle.uniform(18, 4 * 3000).reshape(4, 3000)
    x[0, 2500] = x[0, 17] = 9.0
    x[1, 100] = np.nan
    x[1, 2000] = np.nan
    x[2, 2999] = -9.0
    x[2, 1] = -9.0
    p = Pair.dense(cl, x)
    for d in (0, 1):
        for kind in ("max", "min"):
            wv, wi = oracle.reduce_dim(kind, p.view, d)
            gv, gi = getattr(p.dev, kind)(d + 1)
            assert_bit_equal(gv.float(), wv)
            assert np.array_equal(gi.long(), wi)
    assert p.dev.max(2)[1].long()[0, 0] == 18 and p.dev.max(2)[1].long()[1, 0] == 101
    assert p.dev.min(2)[1].long()[2, 0] == 2


@pytest.mark.parametrize("shape", [(3, 70), (70, 3), (5, 4096), (4096, 8), (300, 260)])
def test_positions_when_every_element_is_the_start_value(cl, shape):
    """max over slices of -inf (min over +inf): nothing ever beats the start
    value, the answer is still position 1; one finite or NaN element moves it."""
    for kind, start in (("max", -np.inf), ("min", np.inf)):
        x = np.full(shape, start, dtype=F)
        x[shape[0] // 2, shape[1] // 2] = 1.0 if kind == "max" else -1.0
        x[shape[0] - 1, 0] = np.nan
        p = Pair.dense(cl, x)
        for d in (0, 1):
            wv, wi = oracle.reduce_dim(kind, p.view, d)
            gv, gi = getattr(p.dev, kind)(d + 1)
            assert_bit_equal(gv.float(), wv, f"{kind} values dim {d + 1}")
            assert np.array_equal(gi.long(), wi), f"{kind} positions dim {d + 1}"
            # untouched slices report position 1
            assert (wi == 1).sum() >= min(shape[1 - d], 2) - 2


@pytest.mark.parametrize("shape,dim0", [((3, 200001), 1), ((200001, 3), 0), ((1, 1 << 19), 1), ((70, 40000), 1), ((40000, 70), 0)])
def test_positions_on_long_slices_cut_over_blocks(cl, shape, dim0):
    """Few long slices are reduced by many blocks whose partial (value, position) pairs are folded afterwards:
    ties keep the lowest position and the first NaN wins, wherever the pieces' borders fall."""
    rs = np.random.RandomState(41)
    R = shape[dim0]
    for mode in ("ties", "nan", "constant"):
        if mode == "ties":
            x = rs.randint(-3, 4, size=shape).astype(F)
        elif mode == "nan":
            x = rs.standard_normal(shape).astype(F)
            for _ in range(4):
                x[tuple(int(rs.randint(n)) for n in shape)] = np.nan
        else:
            x = np.full(shape, F(-1.25))
        X = cl.ClTensor(x)
        rows = np.moveaxis(x, dim0, -1).reshape(-1, R)
        for kind in ("max", "min"):
            want = np.empty(rows.shape[0], dtype=np.int64)
            for k, row in enumerate(rows):
                nans = np.isnan(row)
                want[k] = int(np.argmax(nans)) if nans.any() else int(np.argmax(row) if kind == "max" else np.argmin(row))
            vals, pos = getattr(X, kind)(dim0 + 1)
            got = np.moveaxis(pos.long(), dim0, -1).reshape(-1) - 1
            assert np.array_equal(got, want), (mode, kind)
            got_v = np.moveaxis(vals.float(), dim0, -1).reshape(-1)
            assert_bit_equal(got_v, rows[np.arange(rows.shape[0]), want], f"{mode} {kind} values")
            _, pos64 = getattr(X, f"{kind}_long")(dim0 + 1)
            assert np.array_equal(np.moveaxis(pos64, dim0, -1).reshape(-1) - 1, want)


def test_results_into_existing_strided_tensors(cl):
    x = oracle.uniform(19, 40 * 24).reshape(40, 24)
    X = cl.ClTensor(x)
    holder = Pair.dense(cl, np.zeros((24, 2), dtype=F))
    col = holder.narrow(1, 0, 1).transpose(0, 1)            # sizes (1,24), strides (1,2): right shape, not dense
    st = cl.state()
    import ctypes as C
    st.lib.THClTensor_sum(st.ptr, col.dev._h, X._h, C.c_long(0))
    st.check()
    want = x.astype(np.float64).sum(axis=0).astype(F)
    got = holder.device_storage().reshape(24, 2)
    assert np.array_equal(got[:, 0], want) and np.all(got[:, 1] == 0)


def test_dim_argument_checks(cl):
    X = cl.ClTensor(np.zeros((3, 4), dtype=F))
    with pytest.raises(cl.ClError, match="dimension out of range"):
        X.sum(3)
    with pytest.raises(cl.ClError, match="dimension out of range"):
        X.max(0)
    with pytest.raises(cl.ClError):
        cl.ClTensor(np.zeros(3, dtype=F)).s()              # not a point tensor


def test_profiling_books_launches_under_their_entry_points(cl):
    """cltorch.setProfiling / dumpProfiling (src/init.cpp:149-178)."""
    x = cl.ClTensor(np.ones(1 << 20, dtype=F))
    y = cl.ClTensor(np.ones(1 << 20, dtype=F))
    cl.dumpProfiling()                                   # forget whatever came before
    cl.setProfiling(1)
    for _ in range(5):
        x.add(y)
    x.cmul(y)
    total = x.sum()
    g = cl.ClTensor(np.ones((4096, 64), dtype=F))
    g.sum(1)                                             # a split column reduction: main kernel (+ fold)
    cl.setProfiling(0)
    x.add(y)                                             # not recorded
    report = cl.dumpProfiling()
    rows = {l.split(",")[0]: [float(v) for v in l.split(",")[1:]] for l in report.strip().splitlines()[1:]}
    assert rows["THClTensor_cadd"][0] == 5 and rows["THClTensor_cmul"][0] == 1
    assert rows["THClTensor_sumall"][0] == 1 and rows["THClTensor_sum"][0] >= 1
    assert all(r[1] > 0 and abs(r[2] - r[1] / r[0]) < 1e-3 for r in rows.values())
    assert 0.001 < rows["THClTensor_cadd"][2] < 5.0      # milliseconds per launch: microseconds, not seconds
    assert total == 6.0 * (1 << 20)
    assert cl.dumpProfiling().strip().count("\n") == 0    # records were cleared


@pytest.mark.parametrize("R", [4, 8, 12, 16, 20, 60, 64, 100, 252, 256, 260, 512, 1000, 1024, 2044, 2048])
def test_short_dense_slices_of_every_lane_grouping(cl, R):
    """Dense slices of 4 to 2048 elements (a multiple of 4) take the kernel that shares a slice among 1, 4, 16 or 64
    lanes with one to eight 16-byte loads each and keeps eight passes in flight: slice counts that leave passes and
    blocks ragged, values with ties, NaNs, infinities and slices made of the start value only, outer dims that are
    views (slices start at multiples of 4 elements but are not adjacent), and the value-only kinds."""
    rs = np.random.RandomState(R)
    for n in (1, 3, 257, 5000 if R <= 256 else 700):
        x = rs.randint(-4, 5, size=(n, R)).astype(F)                    # many ties
        x[rs.randint(n), rs.randint(R)] = np.nan
        if n > 2:
            x[1] = -np.inf                                               # a slice made of max's start value
            x[2] = np.inf
            x[2, R - 1] = -np.inf
        p = Pair.dense(cl, x)
        for kind in ("max", "min"):
            wv, wi = oracle.reduce_dim(kind, p.view, 1)
            gv, gi = getattr(p.dev, kind)(2)
            assert_bit_equal(gv.float(), wv, f"{kind} of {n} slices of {R}")
            assert np.array_equal(gi.long(), wi), f"positions of {kind}, {n} slices of {R}"
        y = rs.standard_normal((n, R)).astype(F)
        Y = cl.ClTensor(y)
        close_sum(Y.sum(2).float(), y.astype(np.float64).sum(axis=1, keepdims=True))
        got = Y.prod(2).float() if R <= 64 else None
        if got is not None:
            want = y.astype(np.float64).prod(axis=1, keepdims=True)
            assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-30)
        assert np.allclose(Y.norm(2.0, 2).float(), np.sqrt((y.astype(np.float64) ** 2).sum(axis=1, keepdims=True)), rtol=1e-5)
    # slices that are not adjacent: a narrowed outer dim and a 3-d tensor whose middle dim is narrowed
    z = rs.standard_normal((6, 9, R)).astype(F)
    pz = Pair.dense(cl, z).narrow(1, 2, 5).narrow(0, 1, 4)
    wv, wi = oracle.reduce_dim("max", pz.view, 2)
    gv, gi = pz.dev.max(3)
    assert_bit_equal(gv.float(), wv, "max over the last dim of a narrowed 3-d view")
    assert np.array_equal(gi.long(), wi)
    close_sum(pz.dev.sum(3).float(), z[1:5, 2:7].astype(np.float64).sum(axis=2, keepdims=True))
