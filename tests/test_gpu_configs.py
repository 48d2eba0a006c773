"""The five benchmark configurations at their full sizes, through the C ABI.

Where the CPU oracle finishes in seconds the comparison is direct (bit-exact
for pointwise/copy/positions, 1e-5 relative for sums, 1e-4 for addmm on sampled
entries); the 2^28-element cases add size-independent properties (closed forms,
linearity, idempotence, round trips)."""
import numpy as np
import pytest

import oracle
from oracle import View
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32
EXPR1 = "x = sqrt(1000*x*x + y*10 + z*z)"
EXPR2 = "x = 1000*x + y*10"


def test_config1_contiguous_sequence_2p24(cl):
    n = 1 << 24
    x, y, z = (oracle.uniform(s, n) for s in (1, 2, 3))
    X, Y, Z = cl.ClTensor(x), cl.ClTensor(y), cl.ClTensor(z)
    ref = View.contiguous(x.copy())
    vy, vz = View.contiguous(y), View.contiguous(z)
    X.add(Y)
    oracle.pointwise("cadd", ref, ref, vy, 1.0)
    assert_bit_equal(X.float(), ref.storage, "add")
    X.cmul(Y)
    oracle.pointwise("cmul", ref, ref, vy)
    assert_bit_equal(X.float(), ref.storage, "cmul")
    X.map2_on_gpu(Y, Z, EXPR1)
    oracle.pointwise("map2_c1", ref, vy, vz)
    assert_bit_equal(X.float(), ref.storage, "map2")          # sqrt of negative arguments: NaN on both sides
    assert np.isnan(ref.storage).any()
    # the NaNs make sum and max NaN on both sides (Torch7's CPU rule)
    assert np.isnan(X.sum()) and np.isnan(oracle.sumall(ref))
    assert np.isnan(X.max()) and np.isnan(oracle.maxall(ref))
    # and on NaN-free data they agree numerically
    clean = np.where(np.isnan(ref.storage), F(0), ref.storage)
    C = cl.ClTensor(clean)
    want = oracle.sumall(View.contiguous(clean))
    assert abs(C.sum() - want) <= 1e-5 * abs(want)
    assert C.max() == oracle.maxall(View.contiguous(clean)) and C.min() == oracle.minall(View.contiguous(clean))


def test_config2_strided_views_full_size(cl):
    shape = (512, 512, 256)
    a = Pair.dense(cl, oracle.uniform(4, int(np.prod(shape))).reshape(shape))
    b = Pair.dense(cl, oracle.uniform(5, int(np.prod(shape))).reshape(shape))
    # transpose(1,3) views: sizes (256,512,512), strides (1,256,131072)
    aT, bT = a.transpose(0, 2), b.transpose(0, 2)
    assert aT.dev.size() == (256, 512, 512) and aT.dev.stride() == (1, 256, 131072)
    aT.dev.map_on_gpu(bT.dev, EXPR2)
    oracle.pointwise("map_c2", aT.view, bT.view)
    assert_bit_equal(a.device_storage(), a.host_storage, "map on transposed views")
    # strided copy into a fresh dense destination
    dst = cl.ClTensor(256, 512, 512)
    dst.copy(aT.dev)
    assert_bit_equal(dst.float(), aT.view.gather(), "copy transposed -> dense")
    # stride-2 view: sizes (512,512,128), strides (131072,256,2)
    aS, bS = a.step(2, 2), b.step(2, 2)
    assert aS.dev.stride() == (131072, 256, 2)
    aS.dev.map_on_gpu(bS.dev, EXPR2)
    oracle.pointwise("map_c2", aS.view, bS.view)
    assert_bit_equal(a.device_storage(), a.host_storage, "map on stride-2 views (odd elements untouched)")
    d2 = cl.ClTensor(512, 512, 128)
    d2.copy(aS.dev)
    assert_bit_equal(d2.float(), aS.view.gather(), "copy stride-2 -> dense")
    # narrow view: offset 64, strides (131072,256,1)
    aN, bN = a.narrow(2, 64, 128), b.narrow(2, 64, 128)
    assert aN.dev.storageOffset() == 65
    aN.dev.map_on_gpu(bN.dev, EXPR2)
    oracle.pointwise("map_c2", aN.view, bN.view)
    assert_bit_equal(a.device_storage(), a.host_storage, "map on narrow views")
    # round trip: scatter the dense copy back through the transposed view
    back = Pair.dense(cl, np.zeros(shape, dtype=F))
    back.transpose(0, 2).dev.copy(dst)
    aT_now = dst.float()
    assert_bit_equal(back.transpose(0, 2).dev.float(), aT_now, "dense -> transposed -> read back")
    assert_bit_equal(b.device_storage(), b.host_storage, "inputs untouched")


def test_config3_reductions_along_each_dim_full_size(cl):
    r, c = 4096, 16384
    g = oracle.normal(6, r * c).reshape(r, c)
    p = Pair.dense(cl, g)
    g64 = g.astype(np.float64)
    for dim0 in (0, 1):
        got = p.dev.sum(dim0 + 1).float()
        want = g64.sum(axis=dim0, keepdims=True)
        assert got.shape == want.shape
        # fp64 accumulation on both sides: at most the final rounding to fp32 apart
        assert np.all(np.abs(got - want) <= 1.5 * np.spacing(np.abs(want).astype(F)).astype(np.float64))
        assert np.all(np.abs(got - oracle.reduce_dim("sum", p.view, dim0)[0]) <= np.spacing(np.abs(want).astype(F)))
        for kind in ("max", "min"):
            wv, wi = oracle.reduce_dim(kind, p.view, dim0)
            gv, gi = getattr(p.dev, kind)(dim0 + 1)
            assert_bit_equal(gv.float(), wv, f"{kind} dim {dim0 + 1}")
            assert np.array_equal(gi.long(), wi)
            gv2, gi2 = getattr(p.dev, f"{kind}_long")(dim0 + 1)
            assert np.array_equal(gi2, wi) and gi2.dtype == np.int64
            # the reported position really holds the reported value
            picked = np.take_along_axis(g, gi2 - 1, axis=dim0)
            assert np.array_equal(picked, wv)


def _c4_chain(cl, A, ref):
    """Config 4 on a device tensor and on its host copy with numpy fp32 arithmetic: the sum
    stays on the device as a point tensor, A is divided by it, then 8 further in-place
    operators run with no host synchronisation in between.  Returns the host result."""
    s = cl.ClTensor()
    s.sum(A)                                    # stays on the device
    A.div(s)
    A.mul(1.0001)
    A.add(0.5)
    A.cmul(A)
    A.sqrt()
    s2 = cl.ClTensor()
    s2.max(A)
    A.div(s2)
    A.add(s2)
    A.csub(0.25)
    A.abs()
    cl.synchronize()
    sv, mx = F(s.s()), F(s2.s())
    want_sum = oracle.sumall(View.contiguous(ref))
    assert abs(float(sv) - want_sum) <= 1e-5 * want_sum
    ref /= sv
    ref *= F(1.0001)
    ref += F(0.5)
    ref *= ref
    np.sqrt(ref, out=ref)
    assert mx == ref.max()                      # max of the chain so far, exact
    ref /= mx
    ref += mx
    ref += F(-0.25)
    np.abs(ref, out=ref)
    return ref


def test_config1_sequence_2p28(cl):
    """The same sequence at the size the bandwidth figures are quoted on: add, cmul and the map2 expression over 2^28
    elements compared bit for bit with the dense OpenMP loops of the CPU restatement (a few seconds of host time), then
    sum and max of a copy with the NaNs set to zero against the serial CPU reductions."""
    import ctypes as C
    n = 1 << 28
    L = oracle.lib()
    x, y, z = (oracle.uniform(s, n) for s in (1, 2, 3))
    X, Y, Z = cl.ClTensor(x), cl.ClTensor(y), cl.ClTensor(z)
    p = lambda a: a.ctypes.data_as(C.c_void_p)

    def host(op, val, a, b):          # x = op(a, b), in place in x
        L.th_pointwise_contig_omp(C.c_int(oracle.OPS[op]), C.c_float(val), p(x), p(a), p(b), C.c_long(n))

    X.add(Y)
    host("cadd", 1.0, x, y)
    assert_bit_equal(X.float(), x, "add at 2^28")
    X.cmul(Y)
    host("cmul", 0.0, x, y)
    assert_bit_equal(X.float(), x, "cmul at 2^28")
    X.map2_on_gpu(Y, Z, EXPR1)
    host("map2_c1", 0.0, y, z)
    got = X.float()
    assert_bit_equal(got, x, "map2 at 2^28")
    del got, Y, Z, y, z
    nan = np.isnan(x)
    assert nan.any() and not nan.all()
    assert np.isnan(X.sum()) and np.isnan(X.max())          # Torch7's CPU rule: a NaN decides both
    X.apply_on_gpu("x = (x != x) ? 0.0 : x")
    np.copyto(x, F(0), where=nan)
    v = View.contiguous(x)
    want = oracle.sumall(v)
    assert abs(X.sum() - want) <= 1e-5 * abs(want)
    assert X.max() == oracle.maxall(v) and X.min() == oracle.minall(v)


def test_config4_point_tensor_chain_2p28(cl):
    n = 1 << 28
    a = oracle.uniform(7, n, 0.0, 1.0)
    A = cl.ClTensor(a)
    ref = _c4_chain(cl, A, a.copy())
    got = A.float()
    # every element, so the head, the middle (grid wrap at 2^27) and the tail of the launch are all covered
    for lo, hi in ((0, 1 << 20), ((1 << 27) - (1 << 19), (1 << 27) + (1 << 19)), (n - (1 << 20), n)):
        assert_bit_equal(got[lo:hi], ref[lo:hi], f"chained ops, elements {lo}..{hi}")
    assert_bit_equal(got, ref, "chained ops, all 2^28 elements")
    del got, ref
    # after normalisation the elements sum to 1 (to fp32 rounding of each quotient)
    s = cl.ClTensor()
    A.copy(cl.ClTensor(a))
    s.sum(A)
    A.div(s)
    assert abs(A.sum() - 1.0) < 1e-5
    # closed forms at full size
    A.fill(1.0)
    assert A.sum() == float(n)
    A.fill(0.25)
    assert A.sum() == float(n) * 0.25 and A.max() == 0.25 and A.min() == 0.25
    # max/min bracket every element
    A.copy(cl.ClTensor(a))
    lo, hi = A.min(), A.max()
    assert lo == float(a.min()) and hi == float(a.max())


def test_config4_chain_on_a_misaligned_view_of_2p28_minus_1(cl):
    """The same chain on elements 2..2^28 of the storage: a dense view that starts 4 bytes
    past a 16-byte boundary and whose length is odd, so the dword kernels and their tails run
    at full size.  The element in front of the view must stay untouched."""
    n = 1 << 28
    a = oracle.uniform(7, n, 0.0, 1.0)
    whole = cl.ClTensor(a)
    V = whole.narrow(1, 2, n - 1)
    assert V.storageOffset() == 2 and V.nElement() == n - 1
    ref = _c4_chain(cl, V, a[1:].copy())
    got = whole.float()
    assert got[0] == a[0]
    assert_bit_equal(got[1:], ref, "chained ops on the misaligned view")


def test_config5_addmm_square_8192_sampled_and_skinny(cl):
    n = 8192
    sd = 1.0 / np.sqrt(n)
    a = oracle.normal(8, n * n, 0.0, sd).reshape(n, n)
    b = oracle.normal(9, n * n, 0.0, sd).reshape(n, n)
    c = oracle.normal(10, n * n, 0.0, sd).reshape(n, n)
    got = cl.ClTensor(c).addmm(0.5, 1.0, cl.ClTensor(a), cl.ClTensor(b)).float()
    rng = np.random.RandomState(1)
    rows = np.concatenate([rng.randint(0, n, 4000), [0, 0, n - 1, n - 1, 127, 128]])
    cols = np.concatenate([rng.randint(0, n, 4000), [0, n - 1, 0, n - 1, 128, 127]])
    want = oracle.addmm_f64_sampled(rows, cols, 0.5, View.contiguous(c), 1.0, View.contiguous(a), View.contiguous(b))
    scale = float(np.sqrt(np.mean(want ** 2)))
    assert np.max(np.abs(got[rows, cols] - want)) / scale < 1e-4
    # whole 128x128 output tiles (the kernel's block tile), every entry against fp64 accumulation: the two corners,
    # an interior tile, and the two tiles either side of the seam between the first and second of the eight runs
    # of 512 blocks that the kernel's block renumbering hands to the XCDs (the row-major result is the kernel's
    # column-major one transposed, so its tile (m 7, n 63) is rows 63*128.., columns 7*128.. here)
    for tr, tc in ((0, 0), (63, 63), (29, 41), (63, 7), (0, 8)):
        r0, c0 = tr * 128, tc * 128
        wt = oracle.addmm_f64(0.5, View.contiguous(c[r0:r0 + 128, c0:c0 + 128].copy()), 1.0,
                              View.contiguous(a[r0:r0 + 128].copy()), View.contiguous(b[:, c0:c0 + 128].copy()))
        assert np.max(np.abs(got[r0:r0 + 128, c0:c0 + 128] - wt)) / scale < 1e-4, (tr, tc)
    # checksum of checksums: ones^T (A B) ones == (ones^T A)(B ones), in fp64 from the device result
    lhs = got.astype(np.float64).sum() - 0.5 * c.astype(np.float64).sum()
    rhs = float(a.astype(np.float64).sum(axis=0) @ b.astype(np.float64).sum(axis=1))
    assert abs(lhs - rhs) < 0.05, (lhs, rhs)
    del got
    # skinny: M=64, N=16384, K=4096, A = (K x M dense)^T
    M, N, K = 64, 16384, 4096
    at = oracle.normal(11, K * M, 0.0, sd).reshape(K, M)
    bs = oracle.normal(12, K * N, 0.0, sd).reshape(K, N)
    cs = oracle.normal(13, M * N, 0.0, sd).reshape(M, N)
    pa = Pair.dense(cl, at).transpose(0, 1)
    assert pa.dev.size() == (64, 4096) and pa.dev.stride() == (1, 64)
    pb, pc = Pair.dense(cl, bs), Pair.dense(cl, cs)
    pc.dev.addmm(0.5, 1.0, pa.dev, pb.dev)
    want = oracle.addmm_f64(0.5, pc.view, 1.0, pa.view, pb.view)
    scale = float(np.sqrt(np.mean(want ** 2)))
    assert np.max(np.abs(pc.dev.float() - want)) / scale < 1e-4


def test_dense_tensors_beyond_32_bit_element_counts(cl):
    """The reference caps apply at 2^30 elements (src/lib/THClApply.cpp:136-139).  Dense
    kernels here index with 64 bits: closed forms on 2^31 + 4096 elements (8 GiB
    per tensor), and the strided kernels refuse what their 32-bit indices cannot reach."""
    n = (1 << 31) + 4096
    X, Y = cl.ClTensor(n), cl.ClTensor(n)
    assert X.nElement() == n
    X.fill(1.0)
    Y.fill(2.0)
    X.add(Y)
    assert X.sum() == float(np.float32(3.0 * n))            # fp64 running sum, one rounding
    assert X.max() == 3.0 and X.min() == 3.0
    tail = X.narrow(1, n - 999, 1000)                        # the last elements were reached
    assert tail.float().tolist() == [3.0] * 1000
    X.narrow(1, n - 4, 1).fill(-5.0)                         # a single element past 2^31
    assert X.min() == -5.0 and X.sum() == float(np.float32(3.0 * n - 8.0))
    X.map_on_gpu(Y, "x = x * y")
    assert X.max() == 6.0 and X.min() == -10.0
    half = n // 2
    X.strided((half, 2), (1, half)).add(1.0)                 # a transposed walk over every element: dense after sorting dims
    assert X.max() == 7.0 and X.min() == -9.0



def test_released_blocks_are_reused_without_stalling_or_mixing_owners(cl):
    """The block cache: a tensor's memory goes to the next request of its size while
    the old owner's kernels may still be queued; stream order keeps both right."""
    import os
    if os.environ.get("THCL_ALLOC_CACHE_MB") == "0":
        pytest.skip("the block cache is switched off in this environment")
    n = 1 << 26
    cl.synchronize()
    cl.emptyCache()
    before = cl.memoryStats()
    results = []
    for i in range(12):
        t = cl.ClTensor(n)                       # from the second round on: the block the previous t released
        t.fill(float(i + 1))
        pt = cl.ClTensor()
        pt.sum(t)                                # queued; t is released before it has run
        results.append(pt)
        del t
    after = cl.memoryStats()
    assert [r.s() for r in results] == [float(n) * (i + 1) for i in range(12)]
    assert after["device_mallocs"] - before["device_mallocs"] <= 3 + 12   # one big block (+ the point tensors), not twelve
    assert after["cache_hits"] - before["cache_hits"] >= 11
    assert after["cached_bytes"] >= 4 * n
    # a smaller request may take a block up to a quarter larger, not more
    small = cl.ClTensor(n // 2)
    assert cl.memoryStats()["cached_bytes"] >= 4 * n              # the 256 MiB block was not handed to a 128 MiB request
    del small
    cl.emptyCache()
    assert cl.memoryStats()["cached_bytes"] == 0
    x = cl.ClTensor(n)
    x.fill(2.0)
    assert x.sum() == 2.0 * n


@pytest.mark.parametrize("n", [511, 512, 513, 16383, 16384, 16385, (128 << 8) - 1, 128 << 8, (1 << 18) + 3, (2 << 18) + 1, (9 << 18) - 5, (33 << 18) + 12, (64 << 18), (70 << 18) + 7])
def test_ordinary_host_memory_in_pieces(cl, n):
    """From 2 KiB up, copies from and to ordinary host memory travel in pieces through page-locked buffers with host
    threads copying beside the DMA: lengths on both sides of every piece boundary, both directions, into a fresh array
    and into one that already holds something, float and double hosts, with kernels queued before and after."""
    rng = np.random.RandomState(n % 1000)
    a = rng.standard_normal(n).astype(F)
    t = cl.ClTensor(a)                       # host -> device
    t.mul(2.0)                               # queued behind the upload, ahead of the download
    back = t.float()                         # device -> a new host array
    assert_bit_equal(back, a * F(2.0))
    into = np.full(n, -7.0, dtype=F)
    import ctypes as C
    from cltorch_amd.tensor import _call
    lib = cl.state().lib
    sz = (C.c_long * 1)(n)
    ft = lib.THFloatTensor_newWithData(into.ctypes.data_as(C.c_void_p), n, 0, 1, sz, None)
    try:
        _call("THFloatTensor_copyCl", ft, t._h)
        assert_bit_equal(into, a * F(2.0))
        into[:] = (np.arange(n) % 977).astype(F)
        _call("THClTensor_copyFloat", t._h, ft)          # and back up from the same array
    finally:
        lib.THFloatTensor_free(ft)
    assert t.sum() == float(np.float32(float((np.arange(n) % 977).sum())))
    if n <= (9 << 18):
        d = rng.standard_normal(n)                       # a double host array goes through a float copy first
        s = cl.ClStorage(n)
        s.copy(d)
        assert_bit_equal(s.to_host(), d.astype(F))
        assert np.array_equal(s.to_host(np.float64), d.astype(F).astype(np.float64))


def test_host_threads_and_polling_switched_off(cl):
    """THCL_HOST_COPY_THREADS=0 and THCL_SCALAR_SPIN_US=0 hand the host side back to the embedding process: the
    library starts no thread (float copies go the driver's way, conversions run on the caller) and scalar-returning
    calls wait for the stream instead of polling.  Both are read when the first context is opened, so the
    piece-boundary copies run again in a process of their own (tests/host_side_off_child.py)."""
    import os
    import subprocess
    import sys
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_side_off_child.py")
    env = dict(os.environ, THCL_HOST_COPY_THREADS="0", THCL_SCALAR_SPIN_US="0")
    r = subprocess.run([sys.executable, child], capture_output=True, text=True, env=env, timeout=280)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert "host side off ok" in r.stdout


@pytest.mark.parametrize("n", [(1 << 16) - 1, 1 << 16, (1 << 19) + 5, (3 << 20) + 1, (17 << 20) - 3])
def test_host_arrays_of_other_element_types(cl, n):
    """Dense host arrays of the six other element types: from 65536 elements up they are converted by host threads on
    their way through the page-locked buffers; the values are those of a C cast to float and back, whichever way
    they went.  Storages and LongTensors, lengths on both sides of the switch and of the piece boundaries."""
    rng = np.random.RandomState(n % 997)
    base = rng.standard_normal(n) * 90.0
    for dt in (np.float64, np.int64, np.int32, np.int16, np.int8, np.uint8):
        a = (np.abs(base) if dt == np.uint8 else base).astype(dt)
        s = cl.ClStorage(n)
        s.copy(a)
        want = a.astype(F)
        assert_bit_equal(s.to_host(), want)
        assert np.array_equal(s.to_host(dt), want.astype(dt))
    # LongTensor <-> ClTensor (the host form of index vectors)
    from cltorch_amd.tensor import _call, _long_vector, _LongTensorStruct
    import ctypes as C
    lib = cl.state().lib
    vals = (rng.randint(-10 ** 6, 10 ** 6, size=n)).astype(np.int64)
    lt = _long_vector(vals)
    t = cl.ClTensor(n)
    _call("THClTensor_copyLong", t._h, lt)
    assert_bit_equal(t.float(), vals.astype(F))
    t.add(1.0)
    _call("THLongTensor_copyCl", lt, t._h)
    st = C.cast(lt, C.POINTER(_LongTensorStruct)).contents
    got = np.ctypeslib.as_array(st.storage.contents.data, shape=(n,)).copy()
    lib.THLongTensor_free(lt)
    assert np.array_equal(got, (vals.astype(F) + F(1.0)).astype(np.int64))


def test_pinned_host_arrays(cl):
    """Page-locked host arrays: a round trip through a tensor is exact and views keep the allocation
    alive.  (Transfer rates are a measurement, not a parity property: bench.py reports them.)"""
    n = 1 << 26
    p = cl.pinned_array((n,))
    p[:] = np.arange(n, dtype=F) % 1000
    t = cl.ClTensor(n)
    t.copy(p)
    back = cl.pinned_array((4, n // 4))
    view = back.reshape(-1)
    del back                                            # the view still owns the memory
    import ctypes as C
    from cltorch_amd.tensor import _call
    lib = cl.state().lib

    def d2h(arr):
        sz = (C.c_long * 1)(arr.size)
        ft = lib.THFloatTensor_newWithData(arr.ctypes.data_as(C.c_void_p), arr.size, 0, 1, sz, None)
        try:
            _call("THFloatTensor_copyCl", ft, t._h)
        finally:
            lib.THFloatTensor_free(ft)
    d2h(view)
    assert np.array_equal(view, p)
    pageable = np.zeros(n, dtype=F)
    d2h(pageable)
    assert np.array_equal(pageable, p)
