"""Many launches in a row of every kernel whose blocks hand partial results to one another
(reduce-all dense and strided, dot, the column reduction that folds its splits in the same
launch, the column and row reductions with a finishing kernel, the matrix-vector kernels with
partials, the K-sliced matrix product and the one whose surplus tiles share their K, the single-pass scan
whose blocks hand their totals on while they run), on inputs with closed-form answers: all ones, 1..n,
and a matrix whose column maxima sit at known rows.  Every result of every launch is compared
exactly and the test stops at the first mismatch.  The launches of a round are queued without
waiting in between, so kernels that share tickets and partial slots follow one another the
way a real caller's do."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32
ROUNDS = 80


def test_two_thousand_launches_with_closed_form_results(cl):
    st = {}

    def tensor(key, make):
        if key not in st:
            st[key] = make()
        return st[key]

    n_dense = [(1 << 22) + 5, 1 << 20, 4097, (1 << 24) - 3]
    ones = {n: cl.ClTensor(n).fill(1.0) for n in n_dense}
    ramp_n = 1 << 21
    ramp = cl.ClTensor(np.arange(1, ramp_n + 1, dtype=F))                       # 1..n, every value exact in fp32
    ramp_sum = float(F(ramp_n * (ramp_n + 1) / 2))                              # fp64 running sum is exact, one rounding
    # strided walks: every second element of ones; a narrowed matrix (rows of 100 out of 128)
    strided = ones[1 << 20].strided((1 << 19,), (2,))
    ragged = ones[(1 << 22) + 5].strided((4096, 100), (128, 1))
    # column reductions: 4096 x 8192 folds two splits in the launch; 1<<16 x 1024 folds more; 3000 x 5000 is ragged
    mats = {}
    for (r, c) in ((4096, 8192), (1 << 16, 1024), (3000, 5000)):
        m = cl.ClTensor(r * c).fill(1.0).resize(r, c)
        mats[(r, c)] = m
    # column maxima at known rows: element (r, c) = (r + c) mod R, so column c peaks (value R - 1) at row (R - 1 - c) mod R
    R, Cc = 2048, 4096
    peak = cl.ClTensor(((np.arange(R, dtype=np.int64)[:, None] + np.arange(Cc, dtype=np.int64)[None, :]) % R).astype(F))
    want_rows = ((R - 1 - np.arange(Cc)) % R + 1).astype(np.int64)
    # few long rows (cut over blocks, finished by a second kernel) and a handful of columns
    long_rows = cl.ClTensor(8 << 20).fill(1.0).resize(8, 1 << 20)
    tall = cl.ClTensor(4 << 20).fill(1.0).resize(1 << 20, 4)
    # matrix-vector: ones(4 x 2^22) . ones and its transpose (partials over the contraction), K-sliced product of ones
    mv = cl.ClTensor(4 << 22).fill(1.0).resize(4, 1 << 22)
    vlong, v4 = cl.ClTensor(1 << 22).fill(1.0), cl.ClTensor(4).fill(1.0)
    M, N, K = 64, 4096, 4096
    A, B = cl.ClTensor(M * K).fill(1.0).resize(M, K), cl.ClTensor(K * N).fill(0.5).resize(K, N)
    # 17 x 17 tiles of 128: the 33 tiles beyond the CUs' whole share are computed by several blocks each along K
    T2, K2 = 2176, 512
    A2, B2 = cl.ClTensor(T2 * K2).fill(1.0).resize(T2, K2), cl.ClTensor(K2 * T2).fill(0.5).resize(K2, T2)
    # two rows of 2^23 ones: scanned in one pass by blocks that run together and pass their chunk totals along
    scan_rows = cl.ClTensor(2 << 23).fill(1.0).resize(2, 1 << 23)
    scan_want = np.tile(np.arange(1, (1 << 23) + 1, dtype=F), 2)

    launches = 0
    for rnd in range(ROUNDS):
        checks = []                                                   # (description, device result, expected numpy array)

        def point(src, kind="sum"):
            p = cl.ClTensor()
            getattr(p, kind)(src)
            return p

        for n in n_dense:
            checks.append((f"sum of {n} ones", point(ones[n]), np.array([n], dtype=F)))
            checks.append((f"max of {n} ones", point(ones[n], "max"), np.array([1.0], dtype=F)))
        checks.append(("sum of 1..2^21", point(ramp), np.array([ramp_sum], dtype=F)))
        checks.append(("max of 1..2^21", point(ramp, "max"), np.array([ramp_n], dtype=F)))
        checks.append(("sum of every second one", point(strided), np.array([1 << 19], dtype=F)))
        checks.append(("sum of a narrowed matrix", point(ragged), np.array([409600], dtype=F)))
        for (r, c), m in mats.items():
            checks.append((f"column sums of {r}x{c} ones", m.sum(1), np.full((1, c), r, dtype=F)))
            checks.append((f"row sums of {r}x{c} ones", m.sum(2), np.full((r, 1), c, dtype=F)))
        v, i = peak.max(1)
        checks.append(("column maxima", v, np.full((1, Cc), R - 1, dtype=F)))
        checks.append(("rows of the column maxima", i, want_rows.astype(F).reshape(1, Cc)))
        checks.append(("sums of 8 rows of 2^20", long_rows.sum(2), np.full((8, 1), 1 << 20, dtype=F)))
        checks.append(("column sums of 2^20 x 4", tall.sum(1), np.full((1, 4), 1 << 20, dtype=F)))
        y4, ylong = cl.ClTensor(4).fill(0.0), cl.ClTensor(1 << 22).fill(0.0)
        checks.append(("ones(4 x 2^22) . ones", y4.addmv(0.0, 1.0, mv, vlong), np.full(4, 1 << 22, dtype=F)))
        checks.append(("ones(2^22 x 4) . ones", ylong.addmv(0.0, 1.0, mv.t(), v4), np.full(1 << 22, 4.0, dtype=F)))
        Cm = cl.ClTensor(M, N).fill(1.0)
        checks.append(("K-sliced product of constants", Cm.addmm(0.5, 1.0, A, B), np.full((M, N), 0.5 + K * 0.5, dtype=F)))
        C2 = cl.ClTensor(T2, T2).fill(1.0)
        checks.append(("product whose last tiles share their K", C2.addmm(0.5, 1.0, A2, B2), np.full((T2, T2), 0.5 + K2 * 0.5, dtype=F)))
        if rnd % 4 == 0:
            checks.append(("running sums of two rows of 2^23 ones", scan_rows.cumsum(2), scan_want))
        assert ones[1 << 20].dot(ones[1 << 20]) == float(1 << 20), f"round {rnd}: dot of ones"   # waits for its result
        launches += len(checks) + 5                                 # + the fills above
        cl.synchronize()
        for what, got, want in checks:
            g = got.float().reshape(-1) if got.nDimension() > 0 else np.array([got.s()], dtype=F)
            w = np.asarray(want, dtype=F).reshape(-1)
            bad = np.nonzero(g != w)[0]
            assert bad.size == 0, f"round {rnd}: {what}: {bad.size} wrong, first at {bad[0]}: {g[bad[0]]} instead of {w[bad[0]]}"
    assert launches >= 2000
