"""GPU parity: addmm / gemm against an fp64-accumulated CPU product, 1e-4
relative (measured against the row's magnitude scale), through the C ABI.
Layout cases follow src/lib/THClTensorMathBlas.cpp:107-214."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import View
from gpu_util import Pair

pytestmark = pytest.mark.gpu
F = np.float32
RTOL = 1e-4


def rel_err(got, want):
    """max |got - want| relative to the scale of the result (its RMS), which is
    what a 1e-4 bound on an fp32 dot product of length K can meaningfully mean
    for entries that cancel to nearly zero."""
    want = np.asarray(want, dtype=np.float64)
    scale = max(float(np.sqrt(np.mean(want ** 2))), 1e-30)
    return float(np.max(np.abs(np.asarray(got, dtype=np.float64) - want))) / scale


def test_reference_integer_matrices(cl, golden):
    g = golden["blas_mm"]
    assert cl.mm(cl.ClTensor(g["A"]), cl.ClTensor(g["B"])).float().tolist() == g["expect"]


def _check(cl, pa: Pair, pb: Pair, pc: Pair, beta, alpha):
    want = oracle.addmm_f64(beta, pc.view, alpha, pa.view, pb.view)
    pc.dev.addmm(beta, alpha, pa.dev, pb.dev)
    got = pc.dev.float()
    assert rel_err(got, want) < RTOL
    return got, want


@pytest.mark.parametrize("M,N,K", [(2, 2, 3), (1, 1, 1), (5, 7, 3), (64, 64, 16), (128, 128, 32), (128, 256, 64),
                                   (65, 63, 17), (129, 127, 33), (300, 200, 100), (256, 64, 512), (64, 1024, 48),
                                   (1, 500, 37), (500, 1, 37), (37, 41, 1),
                                   # few tiles and a long K: the K dimension is sliced over blocks
                                   (64, 1024, 2048), (128, 128, 4096), (70, 300, 1500), (33, 65, 5000), (256, 512, 1024)])
def test_shapes_row_major(cl, M, N, K):
    a = oracle.normal(1, M * K).reshape(M, K)
    b = oracle.normal(2, K * N).reshape(K, N)
    c = oracle.normal(3, M * N).reshape(M, N)
    _check(cl, Pair.dense(cl, a), Pair.dense(cl, b), Pair.dense(cl, c), 0.5, 1.0)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("tc", [False, True])
@pytest.mark.parametrize("M,N,K", [(128, 256, 64), (70, 90, 50),
                                   # one row or one column: the matrix-vector kernels; ragged sizes: the edge kernels with
                                   # and without whole 16-byte groups
                                   (1, 3000, 700), (3000, 1, 700), (1, 1, 5000), (1, 64, 4096), (200, 1000, 300), (201, 999, 301),
                                   (32, 32, 40000)])
def test_every_operand_layout(cl, ta, tb, tc, M, N, K):
    """Each operand either dense or the transpose of a dense array: all
    'n'/'t' combinations of the gemm, with the result row- or column-major."""
    a = oracle.normal(4, M * K).reshape(M, K)
    b = oracle.normal(5, K * N).reshape(K, N)
    c = oracle.normal(6, M * N).reshape(M, N)
    pa = Pair.dense(cl, a.T.copy()).transpose(0, 1) if ta else Pair.dense(cl, a)
    pb = Pair.dense(cl, b.T.copy()).transpose(0, 1) if tb else Pair.dense(cl, b)
    pc = Pair.dense(cl, c.T.copy()).transpose(0, 1) if tc else Pair.dense(cl, c)
    got, want = _check(cl, pa, pb, pc, 0.5, 1.5)
    plain = 0.5 * c.astype(np.float64) + 1.5 * (a.astype(np.float64) @ b.astype(np.float64))
    assert np.allclose(want, plain, rtol=1e-12, atol=1e-12)      # the oracle saw the same matrices


def test_operands_with_no_unit_stride_and_gapped_result(cl):
    M, N, K = 48, 40, 24
    a = oracle.normal(7, M * K * 2).reshape(M, K * 2)
    b = oracle.normal(8, K * N * 2).reshape(K, N * 2)
    c = oracle.normal(9, M * N * 2).reshape(M, N * 2)
    pa = Pair.dense(cl, a).step(1, 2)          # strides (2K, 2): neither is 1 -> dense clone inside
    pb = Pair.dense(cl, b).step(1, 2)
    pc = Pair.dense(cl, c).step(1, 2)          # result with neither stride 1 -> computed aside, copied back
    before = pc.host_storage.copy()
    _check(cl, pa, pb, pc, 0.25, 2.0)
    untouched = pc.device_storage().reshape(M, N * 2)[:, 1::2]
    assert np.array_equal(untouched, before.reshape(M, N * 2)[:, 1::2])


def test_beta_zero_ignores_old_contents_and_out_of_place(cl):
    M, N, K = 64, 64, 32
    a = oracle.normal(10, M * K).reshape(M, K)
    b = oracle.normal(11, K * N).reshape(K, N)
    c = np.full((M, N), np.nan, dtype=F)
    got = cl.ClTensor(c).addmm(0.0, 1.0, cl.ClTensor(a), cl.ClTensor(b)).float()
    assert rel_err(got, a.astype(np.float64) @ b.astype(np.float64)) < RTOL
    t = oracle.normal(12, M * N).reshape(M, N)
    T = cl.ClTensor(t)
    r = cl.ClTensor()
    r.addmm(0.5, T, 1.0, cl.ClTensor(a), cl.ClTensor(b))    # r_ != t: t is copied, then updated
    assert rel_err(r.float(), 0.5 * t + a.astype(np.float64) @ b.astype(np.float64)) < RTOL
    assert np.array_equal(T.float(), t)
    with pytest.raises(cl.ClError, match="size mismatch"):
        cl.ClTensor(np.zeros((3, 3), dtype=F)).addmm(cl.ClTensor(a), cl.ClTensor(b))
    with pytest.raises(cl.ClError, match="matrix and matrix expected"):
        cl.ClTensor(c).addmm(cl.ClTensor(np.zeros(4, dtype=F)), cl.ClTensor(b))


def test_gemm_entry_point_column_major(cl):
    # THClBlas_gemm with BLAS argument meaning on column-major data
    m, n, k = 96, 80, 40
    A = oracle.normal(13, m * k).reshape(k, m)      # column-major m x k  == row-major (k, m)
    B = oracle.normal(14, k * n).reshape(n, k)      # column-major k x n
    Cm = oracle.normal(15, m * n).reshape(n, m)     # column-major m x n
    tA, tB, tC = cl.ClTensor(A), cl.ClTensor(B), cl.ClTensor(Cm)
    st = cl.state()
    st.lib.THClBlas_gemm(st.ptr, C.c_char(b"n"), C.c_char(b"n"), m, n, k, C.c_float(1.0), tA._h, m, tB._h, k,
                         C.c_float(0.5), tC._h, m)
    st.check()
    want = 0.5 * Cm.T.astype(np.float64) + A.T.astype(np.float64) @ B.T.astype(np.float64)
    assert rel_err(tC.float().T, want) < RTOL


def test_gemm_with_an_empty_inner_dimension(cl):
    """K = 0 through the BLAS entry point: the result is beta * C (zeros for beta = 0, whatever C held) and the
    operands, which have no elements, are not read."""
    m, n = 70, 45
    Cm = oracle.normal(16, m * n).reshape(n, m)
    Cm[3, 5] = np.nan
    st = cl.state()
    dummy = cl.ClTensor(4)
    for beta in (0.5, 0.0):
        tC = cl.ClTensor(Cm)
        st.lib.THClBlas_gemm(st.ptr, C.c_char(b"n"), C.c_char(b"t"), m, n, 0, C.c_float(2.0), dummy._h, m, dummy._h, n,
                             C.c_float(beta), tC._h, m)
        st.check()
        got = tC.float()
        if beta == 0.0:
            assert np.array_equal(got, np.zeros((n, m), np.float32))
        else:
            assert np.array_equal(got, np.float32(beta) * Cm, equal_nan=True)


def test_skinny_config_shape_reduced(cl):
    # M=64, A given as the transpose of a dense (K x M) array, as in the benchmark configuration
    M, N, K = 64, 2048, 512
    at = oracle.normal(16, K * M, 0.0, 1.0 / np.sqrt(K)).reshape(K, M)
    b = oracle.normal(17, K * N, 0.0, 1.0 / np.sqrt(K)).reshape(K, N)
    c = oracle.normal(18, M * N, 0.0, 1.0 / np.sqrt(K)).reshape(M, N)
    pa = Pair.dense(cl, at).transpose(0, 1)
    assert pa.dev.stride() == (1, 64)
    _check(cl, pa, Pair.dense(cl, b), Pair.dense(cl, c), 0.5, 1.0)


def test_large_square_sampled(cl):
    """2048^3 checked on sampled entries against fp64 dot products, plus a
    size-independent property: (A @ I) == A bit for bit, and linearity in alpha."""
    n = 2048
    a = oracle.normal(8, n * n, 0.0, 1.0 / np.sqrt(n)).reshape(n, n)
    b = oracle.normal(9, n * n, 0.0, 1.0 / np.sqrt(n)).reshape(n, n)
    c = oracle.normal(10, n * n, 0.0, 1.0 / np.sqrt(n)).reshape(n, n)
    A, B = cl.ClTensor(a), cl.ClTensor(b)
    got = cl.ClTensor(c).addmm(0.5, 1.0, A, B).float()
    rng = np.random.RandomState(0)
    rows, cols = rng.randint(0, n, 4096), rng.randint(0, n, 4096)
    want = oracle.addmm_f64_sampled(rows, cols, 0.5, View.contiguous(c), 1.0, View.contiguous(a), View.contiguous(b))
    scale = float(np.sqrt(np.mean(want ** 2)))
    assert np.max(np.abs(got[rows, cols] - want)) / scale < RTOL
    eye = cl.ClTensor(np.eye(n, dtype=F))
    assert np.array_equal(cl.mm(A, eye).float(), a)          # products with 0/1 are exact
    assert np.array_equal(cl.mm(eye, A).float(), a)
    two = cl.ClTensor(np.zeros((n, n), dtype=F)).addmm(0.0, 2.0, A, B).float()
    one = cl.mm(A, B).float()
    assert np.array_equal(two, 2 * one)                      # scaling by 2 is exact


@pytest.mark.parametrize("M,N,K", [(3000, 5000, 208), (1500, 7000, 120), (10000, 2000, 64), (4000, 4000, 104), (3000, 2900, 1000),
                                   (2999, 5001, 77), (6016, 1000, 48)])
def test_ragged_mid_size_shapes(cl, M, N, K):
    """Sizes that are no multiple of the tiles, large enough for the 128-wide edge kernels (whole 16-byte groups, and
    with the odd sizes one element at a time): the whole result against an fp64 product, row- and column-major A."""
    rng = np.random.RandomState(M + N + K)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    want = 0.5 * c.astype(np.float64) + 1.5 * (a.astype(np.float64) @ b.astype(np.float64))
    scale = float(np.sqrt(np.mean(want ** 2)))
    As = (cl.ClTensor(a), cl.ClTensor(np.ascontiguousarray(a.T)).t())
    Bs = (cl.ClTensor(b), cl.ClTensor(np.ascontiguousarray(b.T)).t())
    for A in As:
        for B in Bs:
            got = cl.ClTensor(c).addmm(0.5, 1.5, A, B).float()
            assert np.max(np.abs(got - want)) / scale < RTOL, (A.stride(), B.stride())
    # a column-major result (the product's operands swap roles inside)
    Ct = cl.ClTensor(np.ascontiguousarray(c.T)).t()
    Ct.addmm(0.5, 1.5, As[0], Bs[1])
    assert np.max(np.abs(Ct.float() - want)) / scale < RTOL


@pytest.mark.parametrize("M,N,K", [(16, 300, 128), (300, 16, 128), (32, 256, 64), (256, 32, 64), (1, 1000, 50), (1000, 1, 50),
                                   (7, 129, 33), (129, 7, 33), (32, 4096, 1024), (4096, 24, 2048), (20, 640, 17)])
def test_products_with_a_side_of_at_most_32(cl, M, N, K):
    """A result with at most 32 rows or columns is covered by 128x32 (or 32x128) tiles, four waves side by side along
    the long side: all eight layouts of A, B and the result, whole and ragged sizes, with and without K slicing."""
    rng = np.random.RandomState(M * 7 + N * 3 + K)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    want = 0.5 * c.astype(np.float64) + 2.0 * (a.astype(np.float64) @ b.astype(np.float64))
    scale = max(1.0, float(np.sqrt(np.mean(want ** 2))))
    for lay in range(8):
        A = cl.ClTensor(np.ascontiguousarray(a.T)).t() if lay & 1 else cl.ClTensor(a)
        B = cl.ClTensor(np.ascontiguousarray(b.T)).t() if lay & 2 else cl.ClTensor(b)
        Cd = cl.ClTensor(np.ascontiguousarray(c.T)).t() if lay & 4 else cl.ClTensor(c)
        Cd.addmm(0.5, 2.0, A, B)
        assert np.max(np.abs(Cd.float() - want)) / scale < RTOL, lay


def _odd_pitch(cl, arr, transposed):
    """device tensor equal to arr (2-D), its rows 3 elements apart from dense so that nothing is 16-byte aligned,
    optionally stored transposed"""
    a = np.ascontiguousarray(arr.T if transposed else arr)
    big = np.zeros((a.shape[0], a.shape[1] + 3), F)
    big[:, 1:1 + a.shape[1]] = a
    t = cl.ClTensor(big).narrow(2, 2, a.shape[1])      # the first element sits 4 bytes into the storage
    return t.t() if transposed else t


@pytest.mark.parametrize("M,N,K", [(50, 3, 37), (3, 50, 37), (50, 40, 3), (2, 2, 2), (70, 3, 3), (1, 300, 2), (301, 299, 5),
                                   (129, 131, 67), (1001, 515, 130)])
def test_unaligned_operands_of_any_extent(cl, M, N, K):
    """Operands whose rows start at odd element offsets: 16-byte loads that need no alignment, groups that straddle
    the end of a row or of the operand, fewer than four elements along a row.  All eight layouts."""
    rng = np.random.RandomState(M * 5 + N * 11 + K)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    want = -0.5 * c.astype(np.float64) + 1.25 * (a.astype(np.float64) @ b.astype(np.float64))
    scale = max(1.0, float(np.sqrt(np.mean(want ** 2))))
    for lay in range(8):
        A, B, Cd = _odd_pitch(cl, a, lay & 1), _odd_pitch(cl, b, lay & 2), _odd_pitch(cl, c, lay & 4)
        Cd.addmm(-0.5, 1.25, A, B)
        assert np.max(np.abs(Cd.float() - want)) / scale < RTOL, lay


@pytest.mark.parametrize("M,N,K", [(2176, 2176, 1024), (2100, 2200, 1000), (3072, 3072, 512), (4608, 4608, 300), (2049, 2303, 777),
                                   (2304, 2176, 4100)])
def test_tiles_beyond_a_whole_number_per_cu_share_their_k(cl, M, N, K):
    """A few more 128 x 128 tiles than a multiple of the 256 CUs (289, 306, 576, 1296, 306, 306): the surplus tiles are
    each computed by several blocks along K and summed in slice order.  Whole result against an fp64 product, all four
    layouts of A and B, whole and ragged sizes, beta = 0 over NaNs, and the same bits on a repeat."""
    rng = np.random.RandomState(M + N + K)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    prod = a.astype(np.float64) @ b.astype(np.float64)
    want = 0.5 * c.astype(np.float64) + 1.5 * prod
    scale = float(np.sqrt(np.mean(want ** 2)))
    As = (cl.ClTensor(a), cl.ClTensor(np.ascontiguousarray(a.T)).t())
    Bs = (cl.ClTensor(b), cl.ClTensor(np.ascontiguousarray(b.T)).t())
    for A in As:
        for B in Bs:
            got = cl.ClTensor(c).addmm(0.5, 1.5, A, B).float()
            assert np.max(np.abs(got - want)) / scale < RTOL, (A.stride(), B.stride())
    over_nan = cl.ClTensor(np.full((M, N), np.nan, dtype=F)).addmm(0.0, 1.0, As[0], Bs[0]).float()
    assert np.max(np.abs(over_nan - prod)) / scale < RTOL
    again = cl.ClTensor(np.full((M, N), np.nan, dtype=F)).addmm(0.0, 1.0, As[0], Bs[0]).float()
    assert np.array_equal(over_nan, again)
    Ct = cl.ClTensor(np.ascontiguousarray(c.T)).t()
    Ct.addmm(0.5, 1.5, As[1], Bs[0])
    assert np.max(np.abs(Ct.float() - want)) / scale < RTOL


def _nan_window(cl, arr, transposed, before, after):
    """device tensor equal to arr (2-D): a window of a larger storage that holds NaN everywhere else (`before` rows
    and elements in front of it, `after` behind it), optionally stored transposed"""
    a = np.ascontiguousarray(arr.T if transposed else arr)
    big = np.full((a.shape[0] + before + after, a.shape[1] + before + after), np.nan, F)
    big[before:before + a.shape[0], before:before + a.shape[1]] = a
    t = cl.ClTensor(big).narrow(1, before + 1, a.shape[0]).narrow(2, before + 1, a.shape[1])
    return t.t() if transposed else t


@pytest.mark.parametrize("M,N,K", [(130, 129, 67), (257, 140, 35), (64, 64, 16), (100, 37, 1), (5, 6, 7), (300, 200, 2050),
                                   (96, 1500, 4099), (1030, 1029, 131)])
@pytest.mark.parametrize("before,after", [(1, 2), (4, 0), (0, 0)])
def test_operand_windows_inside_nan_filled_storage(cl, M, N, K, before, after):
    """What lies beside an operand in its storage never reaches the result: tiles on the rim read beyond m and n
    (into the pitch's padding and the neighbouring rows) and the last slab reads beyond k, here all NaN; with
    (0, 0) the operands end exactly where their storage ends.  All eight layouts, K sliced for the longer ones."""
    rng = np.random.RandomState(M * 3 + N * 5 + K * 7)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    want = 0.75 * c.astype(np.float64) + 1.25 * (a.astype(np.float64) @ b.astype(np.float64))
    scale = max(1.0, float(np.sqrt(np.mean(want ** 2))))
    for lay in range(8):
        A, B = _nan_window(cl, a, lay & 1, before, after), _nan_window(cl, b, lay & 2, before, after)
        Cd = cl.ClTensor(np.ascontiguousarray(c.T)).t() if lay & 4 else cl.ClTensor(c)
        Cd.addmm(0.75, 1.25, A, B)
        got = Cd.float()
        assert np.isfinite(got).all(), lay
        assert np.max(np.abs(got - want)) / scale < RTOL, lay


def _long_pitch(cl, arr, transposed, pitch, first):
    """device tensor equal to arr (2-D) whose rows lie `pitch` elements apart in a NaN-filled storage, the first
    one `first` elements into it, optionally stored transposed"""
    a = np.ascontiguousarray(arr.T if transposed else arr)
    store = cl.ClTensor((a.shape[0] - 1) * pitch + a.shape[1] + first).fill(float("nan"))
    t = store.strided(a.shape, (pitch, 1), first + 1)
    t.copy(cl.ClTensor(a))
    return t.t() if transposed else t


@pytest.mark.parametrize("M,N,K", [(5, 6, 7), (70, 3, 3), (130, 129, 67), (40, 260, 150)])
def test_pitches_beyond_the_descriptor_kernels_reach(cl, M, N, K):
    """Rows 2^22 and more elements apart: the tiled kernels with 64-bit addressing, with windows moved back at the
    end of a row and, below four elements along a row, one element at a time.  All four layouts of A and B."""
    rng = np.random.RandomState(M + 2 * N + 3 * K)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    want = 0.5 * c.astype(np.float64) + 1.5 * (a.astype(np.float64) @ b.astype(np.float64))
    scale = max(1.0, float(np.sqrt(np.mean(want ** 2))))
    for lay in range(4):
        A, B = _long_pitch(cl, a, lay & 1, (1 << 22) + 3, 1), _long_pitch(cl, b, lay & 2, 1 << 22, 0)
        got = cl.ClTensor(c).addmm(0.5, 1.5, A, B).float()
        assert np.max(np.abs(got - want)) / scale < RTOL, lay
        del A, B
    cl.emptyCache()


def test_sliced_products_repeat_bit_exactly(cl):
    """K-sliced products sum their slices in slice order: every repetition gives the same
    bits, also with other reductions in between, with ragged shapes, with beta = 0 over
    NaNs, and into a result with gaps between its rows."""
    rng = np.random.RandomState(5)
    for (M, N, K) in ((64, 2048, 4096), (100, 260, 3000), (512, 512, 2048)):
        a = rng.standard_normal((M, K)).astype(F) / np.sqrt(K)
        b = rng.standard_normal((K, N)).astype(F)
        c0 = rng.standard_normal((M, N)).astype(F)
        A, B = cl.ClTensor(a), cl.ClTensor(b)
        want = 0.25 * c0.astype(np.float64) + 2.0 * (a.astype(np.float64) @ b.astype(np.float64))
        first = None
        red = cl.ClTensor(rng.standard_normal((2048, 300)).astype(F))
        red_want = red.float().astype(np.float64).sum(axis=0)
        for rep in range(6):
            Cd = cl.ClTensor(c0)
            Cd.addmm(0.25, 2.0, A, B)
            got = Cd.float()
            assert rel_err(got, want) < RTOL
            if first is None:
                first = got
            assert np.array_equal(first.view(np.uint32), got.view(np.uint32)), (M, N, K, rep)
            s = red.sum(1).float().ravel()
            assert np.allclose(s, red_want, rtol=1e-5, atol=1e-4)
        # beta = 0 never reads the old contents
        Cn = cl.ClTensor(np.full((M, N), np.nan, dtype=F))
        Cn.addmm(0.0, 1.0, A, B)
        assert rel_err(Cn.float(), a.astype(np.float64) @ b.astype(np.float64)) < RTOL
        # rows of the result 8 elements apart from dense: a narrowed view of a wider tensor
        wide = cl.ClTensor(np.zeros((M, N + 8), dtype=F))
        view = wide.narrow(2, 1, N)
        view.copy(cl.ClTensor(c0))
        view.addmm(0.25, 2.0, A, B)
        w = wide.float()
        assert np.array_equal(w[:, :N].view(np.uint32), first.view(np.uint32)) and not w[:, N:].any()


@pytest.mark.parametrize("M,N,K", [(64, 2048, 512), (64, 4096, 1024), (48, 2052, 640), (33, 8192, 514), (32, 4100, 1000), (20, 2048, 4098),
                                   (8, 16384, 768), (4, 3000, 512), (64, 66048, 512), (12, 70000, 520), (64, 16384, 4096)])
def test_short_side_with_a_long_streamed_operand(cl, M, N, K):
    """At most 64 rows (or columns) against a long operand that is contiguous along the long side: the long operand is
    streamed from memory into the matrix cores and only the short one passes through LDS.  Short sides that are no
    multiple of 32 (padded in LDS), long sides that are no multiple of a block's 256 or 512, K that is no multiple of
    a 128-k chunk (the last chunk is short), slices of K and none, both layouts of the short operand, a row-major
    result and the mirrored product into a column-major one, beta = 0 over NaNs, and the same bits on a repeat."""
    rng = np.random.RandomState(M * 13 + N * 3 + K)
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(F)
    b = rng.standard_normal((K, N)).astype(F)
    c = rng.standard_normal((M, N)).astype(F)
    want = 0.5 * c.astype(np.float64) + 1.5 * (a.astype(np.float64) @ b.astype(np.float64))
    scale = float(np.sqrt(np.mean(want ** 2)))
    B = cl.ClTensor(b)
    for A in (cl.ClTensor(a), cl.ClTensor(np.ascontiguousarray(a.T)).t()):
        first = cl.ClTensor(c).addmm(0.5, 1.5, A, B).float()
        assert np.max(np.abs(first - want)) / scale < RTOL, A.stride()
        again = cl.ClTensor(c).addmm(0.5, 1.5, A, B).float()
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
        nan = cl.ClTensor(np.full((M, N), np.nan, dtype=F)).addmm(0.0, 1.0, A, B).float()
        assert np.max(np.abs(nan - a.astype(np.float64) @ b.astype(np.float64))) / scale < RTOL
        # mirrored: (N x K) @ (K x M) into a column-major result, the long operand given as the transpose of a dense array
        Ct = cl.ClTensor(np.ascontiguousarray(c)).t()                 # N x M with strides (1, N)
        Ct.addmm(0.5, 1.5, B.t(), A.t())
        assert np.max(np.abs(Ct.float().T - want)) / scale < RTOL, ("mirrored", A.stride())
