"""cumsum / cumprod, mean, norms and all / any through the C ABI against
oracle/catalogue.py (Torch7 CPU semantics: fp64 running values).  Scans: the
device combines fp64 partial results in a different order than the sequential
oracle, so an output may land on the neighbouring fp32 value when the fp64
result sits within 1e-16 of a rounding boundary: the bar is <= 1 ulp everywhere
and bit-equality for at least 99.99 % of the elements."""
import numpy as np
import pytest

import oracle
from oracle import catalogue as cat
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32


def _scan_close(got, want, what):
    assert got.shape == want.shape, what
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.mean() >= 0.9999, f"{what}: only {same.mean():.6f} bit-equal"
    bad = ~same
    if bad.any():
        assert np.all(np.abs(got[bad] - want[bad]) <= np.spacing(np.abs(want[bad]))), f"{what}: more than 1 ulp"


SHAPES = [(1,), (5,), (1023,), (1024,), (4099,), (300000,), (7, 5), (3, 2000), (2000, 3), (64, 4096), (33, 70, 9),
          (4, 300, 128), (2, 3, 4, 5), (1, 50000), (50000, 1), (6, 1 << 16),
          (5000, 2), (5000, 3), (3000, 16), (3000, 18), (700, 100), (700, 256), (300, 1000), (20000, 2048), (9, 7, 130),
          (1000, 16384), (777, 8200), (3, 700, 4096), (513, 32768),
          # outer scans of 1024 rows and more over strips of 32 columns, and of 64 where those give every CU a block
          # (whole and ragged last strips, one and two outer slices)
          (1030, 8192), (1100, 16384), (1500, 16400), (2, 1100, 8200), (1025, 4100), (2600, 16384),
          # a handful of columns and long lines: strips as wide as the tensor, lines cut into segments
          (1 << 20, 4), (300001, 8), (100003, 12), (70000, 28), (3, 40000, 8), (2, 20000, 20), (16384, 16)]


@pytest.mark.parametrize("shape", SHAPES)
def test_cumsum_every_dim(cl, shape):
    x = oracle.uniform(61, int(np.prod(shape))).reshape(shape)
    X = cl.ClTensor(x)
    for d in range(len(shape)):
        _scan_close(X.cumsum(d + 1).float(), cat.cumulate(x, d), f"cumsum {shape} dim {d + 1}")


@pytest.mark.parametrize("shape", [(37,), (5000,), (40, 300), (300, 40), (9, 33, 17), (600, 8200), (50000, 4), (2, 30000, 12),
                                   (1200, 16384), (1040, 8200)])
def test_cumprod_every_dim(cl, shape):
    x = oracle.uniform(62, int(np.prod(shape)), 0.9, 1.1)
    x[::7] *= -1
    x = x.reshape(shape)
    X = cl.ClTensor(x)
    for d in range(len(shape)):
        _scan_close(X.cumprod(d + 1).float(), cat.cumulate(x, d, prod=True), f"cumprod {shape} dim {d + 1}")


@pytest.mark.parametrize("shape,prod", [(((1 << 24) + 4096,), False), (((1 << 25) + 8200 * 4,), False), ((3, 1 << 24), False),
                                        (((1 << 24) + 12,), True), ((1 << 27,), False),
                                        ((64, 1 << 20), False), ((5, (1 << 22) + 4000), False), ((256, 1 << 16), False),
                                        ((700, 30000), False), ((2, 3, (1 << 22) - 8), True), ((767, 21880), False)])
def test_long_rows_in_one_pass(cl, shape, prod):
    """2^24 elements and more in rows (a multiple of 4 long, aligned) that are too few for a block each are scanned in
    one pass by blocks that hand their totals on while they run: whole and ragged last chunks and rounds, one row and
    several hundred (a row's chunks in one round, across rounds, rows that begin in the middle of a round), sums and
    products."""
    n = int(np.prod(shape))
    x = (oracle.uniform(71, n, 0.9995, 1.0005) if prod else oracle.uniform(72, n)).reshape(shape)
    X = cl.ClTensor(x)
    d = len(shape)
    got = (X.cumprod(d) if prod else X.cumsum(d)).float()
    _scan_close(got, cat.cumulate(x, d - 1, prod=prod), f"long rows {shape}")
    if not prod and len(shape) == 1:
        ones = cl.ClTensor(n)
        ones.fill(1.0)
        assert np.array_equal(ones.cumsum().float(), np.arange(1, n + 1, dtype=np.float64).astype(F))   # exact below 2^24, rounded above


def test_single_pass_scan_gives_up_instead_of_hanging(cl):
    """A block of the single-pass scan that never publishes its totals (forced from the host, with waits that poll
    once): every kernel still ends, the failure is reported at the next wait and the library keeps working
    (tests/scan_give_up_child.py, in a process of its own because both switches are read once)."""
    import os
    import subprocess
    import sys
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scan_give_up_child.py")
    env = dict(os.environ, THCL_SCAN_CHAIN_SPINS="0", THCL_SCAN_CHAIN_MUTE="0")
    r = subprocess.run([sys.executable, child], capture_output=True, text=True, env=env, timeout=110)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "scan give-up ok" in r.stdout


def test_scan_closed_forms_views_and_in_place(cl):
    n = 1 << 22                                             # long row: segments + carries
    ones = cl.ClTensor(n)
    ones.fill(1.0)
    got = ones.cumsum().float()
    assert np.array_equal(got, np.arange(1, n + 1, dtype=np.float64).astype(F))   # exact: fp64 running value
    big = cl.ClTensor(np.array([16777216.0, 1.0, 1.0, 1.0], dtype=F))
    assert big.cumsum().float().tolist() == [16777216.0, 16777216.0, 16777218.0, 16777220.0]
    twos = cl.ClTensor(30)
    twos.fill(2.0)
    assert np.array_equal(twos.cumprod().float(), (2.0 ** np.arange(1, 31)).astype(F))
    # strided source and destination
    x = oracle.uniform(63, 60 * 50).reshape(60, 50)
    p = Pair.dense(cl, x).transpose(0, 1)
    for d in (0, 1):
        _scan_close(p.dev.cumsum(d + 1).float(), cat.cumulate(p.view.gather(), d), f"transposed source dim {d + 1}")
    dst = Pair.dense(cl, np.zeros((50, 60), dtype=F)).transpose(0, 1)      # 60 x 50 view of a 50 x 60 storage
    dst.dev.cumsum(Pair.dense(cl, x).dev, 1)
    _scan_close(dst.dev.float(), cat.cumulate(x, 0), "strided destination")
    same = cl.ClTensor(x)
    same.cumsum(same, 2)                                   # result and source are one tensor
    _scan_close(same.float(), cat.cumulate(x, 1), "in place")
    with pytest.raises(cl.ClError):
        cl.ClTensor(x).cumsum(3)


def test_scan_of_long_rows(cl):
    """Rows too few to fill the chip are cut into segments: segment totals, a scan of the totals, then the
    scan proper.  2^25 + 5000 elements end in a ragged segment; the result is the same on every run."""
    n = (1 << 25) + 5000
    ones = cl.ClTensor(n)
    ones.fill(1.0)
    assert np.array_equal(ones.cumsum().float(), np.arange(1, n + 1, dtype=np.float64).astype(F))
    x = oracle.uniform(66, n)
    X = cl.ClTensor(x)
    first = X.cumsum().float()
    _scan_close(first, cat.cumulate(x, 0), "cumsum of 2^25 + 5000 elements")
    for _ in range(3):
        assert_bit_equal(X.cumsum().float(), first, "repeat of the same scan")
    # an odd length and a source that starts 4 bytes off a 16-byte boundary: the scalar path
    xo = X.narrow(1, 2, n - 2)
    _scan_close(xo.cumsum().float(), cat.cumulate(x[1:n - 1], 0), "unaligned source")
    # three long rows; products that stay near 1
    y = oracle.uniform(67, 3 * 70 * 4096, 0.999, 1.001).reshape(3, 70 * 4096)
    _scan_close(cl.ClTensor(y).cumprod(2).float(), cat.cumulate(y, 1, prod=True), "cumprod of 3 long rows")
    _scan_close(cl.ClTensor(y).cumsum(2).float(), cat.cumulate(y, 1), "cumsum of 3 long rows")


def test_mean_and_norms(cl):
    x = oracle.normal(64, 300 * 700).reshape(300, 700)
    x[5, :40] = 0.0
    X = cl.ClTensor(x)
    x64 = x.astype(np.float64)
    assert abs(X.mean() - x64.mean()) <= 1e-5 * abs(x64.mean()) + 1e-7
    for d in (0, 1):
        got = X.mean(d + 1).float()
        want = (x64.sum(axis=d, keepdims=True).astype(F) / F(x.shape[d])).astype(F)   # fp32 sum, then one division
        assert_bit_equal(got, want, f"mean dim {d + 1}")
    for p in (0.0, 1.0, 2.0, 3.0, 0.5, 2.5):
        want = float(cat.norm(x, p))
        assert abs(X.norm(p) - want) <= 1e-5 * want, (p, X.norm(p), want)
        for d in (0, 1):
            got = X.norm(p, d + 1).float()
            wd = cat.norm(x, p, axis=d)
            assert got.shape == wd.shape
            assert np.all(np.abs(got - wd) <= 1e-5 * np.abs(wd) + 1e-30), (p, d)
    assert X.norm() == X.norm(2.0)                          # default exponent
    assert X.norm(0.0) == float((x != 0).sum())             # exact count
    t = Pair.dense(cl, x).transpose(0, 1).narrow(0, 3, 500)
    want = float(cat.norm(t.view.gather(), 2.0))
    assert abs(t.dev.norm(2.0) - want) <= 1e-5 * want
    with pytest.raises(cl.ClError):
        cl.ClTensor().mean()


def test_all_any(cl):
    n = 1 << 20
    x = oracle.uniform(65, n, 1.0, 5.0)
    X = cl.ClTensor(x)
    assert X.all() is True and X.any() is True
    x2 = x.copy()
    x2[n - 7] = 0.5                                         # (int)0.5 == 0: false for the reference's all
    assert cl.ClTensor(x2).all() is False and bool(cat.truth(x2).all()) is False
    z = np.zeros(n, dtype=F)
    assert cl.ClTensor(z).any() is False and cl.ClTensor(z).all() is False
    z[12345] = -3.0
    assert cl.ClTensor(z).any() is True
    z[12345] = 0.99
    assert cl.ClTensor(z).any() is False and bool(cat.truth(z).any()) is False
    pt = cl.ClTensor()
    pt.all(X)
    assert pt.nDimension() == 0 and pt.s() == 1.0
    pt.any(cl.ClTensor(np.zeros(100, dtype=F)))
    assert pt.s() == 0.0
    s = Pair.dense(cl, x2.reshape(1024, 1024)).transpose(0, 1).narrow(1, 0, 1000)   # drops row 1023 with the 0.5
    assert s.dev.all() is bool(cat.truth(s.view.gather()).all())


@pytest.mark.parametrize("rows,cols,skip", [(600000, 3, 0), (300000, 7, 0), (200000, 10, 0), (70000, 27, 0), (300000, 6, 1), (250000, 8, 1),
                                            (400000, 4, 0), (20000, 5, 0)])
def test_scans_down_a_few_columns(cl, rows, cols, skip):
    """Long scans down 3 to 27 columns: strips as wide as the tensor, with whole 16-byte groups where the width and
    the rows' alignment allow (skip = rows dropped in front, which shifts the alignment), one element at a time
    otherwise; short tensors take the thread-per-column walk."""
    x = oracle.uniform(200 + cols, (rows + skip) * cols).reshape(rows + skip, cols)
    X = cl.ClTensor(x)
    V = X.narrow(1, skip + 1, rows) if skip else X
    xv = x[skip:]
    _scan_close(V.cumsum(1).float(), cat.cumulate(xv, 0), f"cumsum {rows} x {cols}")
    y = (1.0 + 1e-5 * xv).astype(F)
    Y = cl.ClTensor(y)
    Y.cumprod(Y, 1)
    _scan_close(Y.float(), cat.cumulate(y, 0, prod=True), "cumprod in place")
    ones = cl.ClTensor(np.ones((rows, cols), dtype=F))
    assert np.array_equal(ones.cumsum(1).float()[:, cols - 1], np.arange(1, rows + 1, dtype=F))


@pytest.mark.parametrize("rows,length", [(4200, 1028), (4100, 2048), (4096, 3000), (5000, 1024), (4300, 8188)])
def test_many_rows_of_a_thousand_to_eight_thousand_elements(cl, rows, length):
    """Enough aligned rows for a wave each: whole batches of 1024 elements plus a ragged rest, out of place, in
    place, and as products."""
    x = oracle.uniform(91 + length, rows * length).reshape(rows, length)
    X = cl.ClTensor(x)
    _scan_close(X.cumsum(2).float(), cat.cumulate(x, 1), f"cumsum {rows} x {length}")
    Y = cl.ClTensor(x)
    Y.cumsum(Y, 2)
    _scan_close(Y.float(), cat.cumulate(x, 1), "in place")
    y = (1.0 + 0.001 * x).astype(F)
    _scan_close(cl.ClTensor(y).cumprod(2).float(), cat.cumulate(y, 1, prod=True), "cumprod")
    ones = cl.ClTensor(np.ones((rows, length), dtype=F))
    assert np.array_equal(ones.cumsum(2).float()[rows - 1], np.arange(1, length + 1, dtype=F))


def test_scan_of_rows_longer_than_a_window(cl):
    """Cut rows of more than 128 MiB in total go through in windows (totals pass and scan pass per window), and a
    segment's carry-in comes partly from the previous window's last block, partly from the window's own totals:
    rows that begin, end and straddle a window boundary, checked on ones (every prefix is a count) and on a ramp
    of small integers (every prefix exact in fp64), plus run-to-run equality on random data."""
    for rows, length in ((1, (1 << 26) + 12288 + 4), (3, (1 << 25) + 20480), (64, 1 << 20), (5, 9 * (1 << 20) + 4096)):
        ones = cl.ClTensor(rows * length).fill(1.0).resize(rows, length)
        got = ones.cumsum(2).float()
        want = np.arange(1, length + 1, dtype=np.float64).astype(F)
        for r in range(rows):
            assert np.array_equal(got[r], want), (rows, length, r)
        del ones, got
    n = (1 << 26) + 4096 * 3
    ramp = (np.arange(n, dtype=np.int64) % 7).astype(F)
    got = cl.ClTensor(ramp).cumsum().float()
    assert np.array_equal(got, np.cumsum(ramp.astype(np.float64)).astype(F))
    x = oracle.uniform(68, n)
    X = cl.ClTensor(x)
    first = X.cumsum().float()
    _scan_close(first, cat.cumulate(x, 0), "cumsum across windows")
    assert_bit_equal(X.cumsum().float(), first, "repeat of the same scan")
    y = oracle.uniform(69, n, 0.9999999, 1.0000001)
    _scan_close(cl.ClTensor(y).cumprod().float(), cat.cumulate(y, 0, prod=True), "cumprod across windows")
