"""indexSelect / indexCopy / indexFill, gather / scatter, maskedSelect /
maskedCopy through the C ABI against oracle/catalogue.py.  Pure data movement:
every comparison is bit for bit."""
import numpy as np
import pytest

import oracle
from oracle import catalogue as cat
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32


def _rng(seed):
    return np.random.RandomState(seed)


@pytest.mark.parametrize("shape,dim", [((7,), 0), ((50, 64), 0), ((50, 64), 1), ((33, 17), 0), ((33, 17), 1),
                                       ((6, 40, 12), 1), ((5, 9, 260), 0), ((5, 9, 260), 2), ((3000, 128), 0),
                                       ((2, 3, 4, 5), 2)])
def test_index_select_copy_fill(cl, shape, dim):
    n = int(np.prod(shape))
    x = oracle.uniform(101, n).reshape(shape)
    X = cl.ClTensor(x)
    r = _rng(dim + n)
    m = max(1, shape[dim] // 2 + 3)
    idx = r.randint(1, shape[dim] + 1, size=m)                      # repeats allowed
    # select: device float indices, host long indices
    want = cat.index_select(x, dim, idx)
    assert_bit_equal(X.index(dim + 1, cl.ClTensor(idx.astype(F))).float(), want, "indexSelect")
    assert_bit_equal(X.index(dim + 1, idx.tolist()).float(), want, "indexSelect_long")
    # copy: repeated targets keep the last source slice
    srcshape = list(shape)
    srcshape[dim] = m
    src = oracle.uniform(102, int(np.prod(srcshape))).reshape(srcshape)
    R = cl.ClTensor(x)
    R.indexCopy(dim + 1, cl.ClTensor(idx.astype(F)), cl.ClTensor(src))
    assert_bit_equal(R.float(), cat.index_copy(x, dim, idx, src), "indexCopy")
    R2 = cl.ClTensor(x)
    R2.indexCopy(dim + 1, idx, cl.ClTensor(src))
    assert_bit_equal(R2.float(), cat.index_copy(x, dim, idx, src), "indexCopy_long")
    # fill
    R3 = cl.ClTensor(x)
    R3.indexFill(dim + 1, cl.ClTensor(idx.astype(F)), -7.0)
    assert_bit_equal(R3.float(), cat.index_fill(x, dim, idx, -7.0), "indexFill")
    R4 = cl.ClTensor(x)
    R4.indexFill(dim + 1, idx[:1], 3.0)
    assert_bit_equal(R4.float(), cat.index_fill(x, dim, idx[:1], 3.0), "indexFill_long")


def test_index_ops_on_views_and_bad_arguments(cl):
    x = oracle.uniform(103, 40 * 30).reshape(40, 30)
    p = Pair.dense(cl, x).transpose(0, 1)                            # 30 x 40, strides (1, 30)
    idx = np.array([5, 1, 30, 5, 2])
    got = p.dev.index(1, cl.ClTensor(idx.astype(F)))
    assert_bit_equal(got.float(), cat.index_select(p.view.gather(), 0, idx), "select from a transposed view")
    dst = Pair.dense(cl, np.zeros((40, 30), dtype=F)).transpose(0, 1)
    src = oracle.uniform(104, 5 * 40).reshape(5, 40)
    dst.dev.indexCopy(1, cl.ClTensor(idx.astype(F)), cl.ClTensor(src))
    assert_bit_equal(dst.dev.float(), cat.index_copy(np.zeros((30, 40), dtype=F), 0, idx, src), "copy into a transposed view")
    dst.dev.indexFill(2, [1, 40], 9.0)
    assert np.all(dst.dev.float()[:, [0, 39]] == 9.0)
    # an index outside the dimension moves nothing and is reported as an error at the next wait for the device
    # (Torch's CPU path raises at once; the reference's kernels read or write out of bounds)
    Y = cl.ClTensor(x)
    sel = Y.index(1, cl.ClTensor(np.array([1, 41, 0, 40], dtype=F)))
    with pytest.raises(cl.ClError, match="index out of range"):
        cl.synchronize()
    assert_bit_equal(sel.float()[[0, 3]], x[[0, 39]], "valid rows")           # the report is made once; the library goes on
    Y.indexFill(1, cl.ClTensor(np.array([0, 41, -3], dtype=F)), 5.0)
    with pytest.raises(cl.ClError, match="index out of range"):
        Y.float()                                                              # a read-back waits too
    assert_bit_equal(Y.float(), x, "out-of-range fill is a no-op")
    gi = np.ones((1, 30), dtype=F)
    gi[0, 7] = 99.0
    g = cl.ClTensor(x).gather(1, cl.ClTensor(gi))
    with pytest.raises(cl.ClError, match="index out of range"):
        cl.synchronize()
    del g
    Z = cl.ClTensor(x)
    Z.indexCopy(1, cl.ClTensor(np.array([2, float("nan")], dtype=F)), cl.ClTensor(x[:2] * 0 + 1))
    with pytest.raises(cl.ClError, match="index out of range"):
        cl.synchronize()
    assert np.all(Z.float()[1] == 1.0) and np.array_equal(Z.float()[[0, 2]], x[[0, 2]])
    cl.synchronize()                                                           # nothing pending any more
    with pytest.raises(cl.ClError):
        Y.index(3, [1])
    with pytest.raises(cl.ClError):
        Y.index(1, cl.ClTensor(np.ones((2, 2), dtype=F)))
    with pytest.raises(cl.ClError):
        Y.indexCopy(1, [1, 2, 3], cl.ClTensor(2, 30))


@pytest.mark.parametrize("shape,dim", [((6, 5), 0), ((6, 5), 1), ((40, 300), 0), ((40, 300), 1), ((7, 30, 20), 1),
                                       ((3, 4, 5, 6), 3), ((2000, 64), 0)])
def test_gather_scatter(cl, shape, dim):
    n = int(np.prod(shape))
    x = oracle.uniform(105, n).reshape(shape)
    r = _rng(n + dim)
    ishape = list(shape)
    ishape[dim] = max(1, shape[dim] // 2)
    index = r.randint(1, shape[dim] + 1, size=ishape)
    X, I = cl.ClTensor(x), cl.ClTensor(index.astype(F))
    assert_bit_equal(X.gather(dim + 1, I).float(), cat.gather(x, dim, index), "gather")
    # scatter needs distinct targets along dim for a defined result: a permutation prefix per line
    perm = np.argsort(r.rand(*shape), axis=dim) + 1
    take = [slice(None)] * len(shape)
    take[dim] = slice(0, ishape[dim])
    uidx = perm[tuple(take)]
    src = oracle.uniform(106, int(np.prod(ishape))).reshape(ishape)
    R = cl.ClTensor(x)
    R.scatter(dim + 1, cl.ClTensor(uidx.astype(F)), cl.ClTensor(src))
    assert_bit_equal(R.float(), cat.scatter(x, dim, uidx, src), "scatter")
    R2 = cl.ClTensor(x)
    R2.scatter(dim + 1, cl.ClTensor(uidx.astype(F)), 2.5)
    assert_bit_equal(R2.float(), cat.scatter(x, dim, uidx, 2.5), "scatterFill")
    # round trip
    back = R.gather(dim + 1, cl.ClTensor(uidx.astype(F)))
    assert_bit_equal(back.float(), src, "gather undoes scatter")


def test_gather_scatter_views_and_checks(cl):
    x = oracle.uniform(107, 30 * 20).reshape(30, 20)
    p = Pair.dense(cl, x).transpose(0, 1)                            # 20 x 30
    index = _rng(5).randint(1, 21, size=(4, 30))
    pi = Pair.dense(cl, index.T.astype(F)).transpose(0, 1)           # a strided index tensor
    assert_bit_equal(p.dev.gather(1, pi.dev).float(), cat.gather(p.view.gather(), 0, index), "gather on views")
    X = cl.ClTensor(x)
    with pytest.raises(cl.ClError):
        X.gather(1, cl.ClTensor(np.ones((2, 19), dtype=F)))          # other dims must match
    with pytest.raises(cl.ClError):
        X.gather(3, cl.ClTensor(np.ones((2, 20), dtype=F)))
    with pytest.raises(cl.ClError):
        X.scatter(1, cl.ClTensor(np.ones((2, 20), dtype=F)), cl.ClTensor(3, 20))


@pytest.mark.parametrize("n", [1, 2, 3, 5, 6, 255, 256, 1023, 1025, 4095, 4096, 4097, 100003, (1 << 22) + 11, (1 << 24) + 3 * 4099])
def test_masked_select_and_copy(cl, n):
    x = oracle.uniform(108, n)
    mask = (oracle.uniform(109, n) > 0.2).astype(F)
    mask[::97] *= -3.0                                              # any non-zero selects
    X, M = cl.ClTensor(x), cl.ClTensor(mask)
    got = X.maskedSelect(M)
    want = cat.masked_select(x, mask)
    assert got.nDimension() == 1 and got.size() == (want.size,)
    assert_bit_equal(got.float(), want, "maskedSelect")
    src = oracle.uniform(110, max(1, want.size))
    if want.size:
        R = cl.ClTensor(x)
        R.maskedCopy(M, cl.ClTensor(src))
        assert_bit_equal(R.float(), cat.masked_copy(x, mask, src), "maskedCopy")
        # select undoes copy
        assert_bit_equal(R.maskedSelect(M).float(), src[:want.size], "round trip")


def test_masked_edge_cases(cl):
    n = 10000
    x = oracle.uniform(111, n)
    X = cl.ClTensor(x)
    none = X.maskedSelect(cl.ClTensor(np.zeros(n, dtype=F)))
    assert none.nElement() == 0 and none.nDimension() == 0 and none.float().shape == (0,)
    every = X.maskedSelect(cl.ClTensor(np.ones(n, dtype=F)))
    assert_bit_equal(every.float(), x, "all selected")
    # 2-d strided source and mask
    p = Pair.dense(cl, x.reshape(100, 100)).transpose(0, 1)
    m = (oracle.uniform(112, n) > 0.0).astype(F).reshape(100, 100)
    assert_bit_equal(p.dev.maskedSelect(cl.ClTensor(m)).float(), cat.masked_select(p.view.gather(), m), "strided source")
    # operands that start 4 bytes off a 16-byte boundary: the scalar path
    xo, mo = X.narrow(1, 2, n - 1), cl.ClTensor(m.reshape(-1)).narrow(1, 2, n - 1)
    assert_bit_equal(xo.maskedSelect(mo).float(), cat.masked_select(x[1:], m.reshape(-1)[1:]), "unaligned operands")
    with pytest.raises(cl.ClError):
        X.maskedSelect(cl.ClTensor(n + 1))
    R = cl.ClTensor(x)
    with pytest.raises(cl.ClError, match="source nElements"):
        R.maskedCopy(cl.ClTensor(np.ones(n, dtype=F)), cl.ClTensor(n - 1))


def test_host_element_types_and_byte_masks(cl):
    """copyByte/Char/Short/Int/Double both ways (src/lib/THClTensorCopy.h:8-22) and the
    byte-mask forms of the masked operators (src/lib/THClTensorMasked.cpp:248-281)."""
    vals = np.array([[0, 1, 2.75, -3.5], [100, -128, 127, 255], [65000.5, -7, 8, 9]], dtype=F)
    X = cl.ClTensor(vals)
    assert np.array_equal(X.double(), vals.astype(np.float64)) and X.double().dtype == np.float64
    assert np.array_equal(X.int(), vals.astype(np.int32))                 # C conversion: truncation toward zero
    small = cl.ClTensor(np.array([[0, 1, 2.75], [-3.5, 100, 127]], dtype=F))
    assert np.array_equal(small.short(), np.array([[0, 1, 2], [-3, 100, 127]], dtype=np.int16))
    assert np.array_equal(small.char(), np.array([[0, 1, 2], [-3, 100, 127]], dtype=np.int8))
    pos = cl.ClTensor(np.array([0, 1, 2.75, 200, 255], dtype=F))
    assert np.array_equal(pos.byte(), np.array([0, 1, 2, 200, 255], dtype=np.uint8))
    for dtype in (np.uint8, np.int8, np.int16, np.int32, np.float64):
        h = (np.arange(24).reshape(4, 6) % 100).astype(dtype)
        T = cl.ClTensor(4, 6)
        T.copyFrom(h)
        assert_bit_equal(T.float(), h.astype(F), f"from {dtype.__name__}")
        T2 = cl.ClTensor(6, 4)
        T2.copyFrom(h.T)                                                  # strided host view
        assert_bit_equal(T2.float(), h.T.astype(F), f"from transposed {dtype.__name__}")
        dst = Pair.dense(cl, np.zeros((6, 4), dtype=F)).transpose(0, 1)   # strided device view
        dst.dev.copyFrom(h)
        assert_bit_equal(dst.dev.float(), h.astype(F), f"into a transposed view from {dtype.__name__}")
    d = np.array([1e-3, 1.0000001, 16777217.0, -2.5e38], dtype=np.float64)
    D = cl.ClTensor(4)
    D.copyFrom(d)
    assert_bit_equal(D.float(), d.astype(F), "double -> float rounding")
    with pytest.raises(cl.ClError):
        cl.ClTensor(5).copyFrom(np.zeros(4, dtype=np.int32))
    # byte masks
    x = oracle.uniform(121, 5000).reshape(50, 100)
    m = oracle.uniform(122, 5000).reshape(50, 100) > 0.1
    Xm = cl.ClTensor(x)
    assert_bit_equal(Xm.maskedSelect(m).float(), cat.masked_select(x, m), "maskedSelectByte")
    Xm.maskedFill(m, 4.0)
    assert_bit_equal(Xm.float(), cat.masked_fill(x, m, 4.0), "maskedFillByte")
    src = oracle.uniform(123, int(m.sum()))
    Xc = cl.ClTensor(x)
    Xc.maskedCopy(m, cl.ClTensor(src))
    assert_bit_equal(Xc.float(), cat.masked_copy(x, m, src), "maskedCopyByte")


def test_header_and_storage_interface_extras(cl):
    """resize5d, squeeze1d, 3-d / 4-d element access, whole-storage copies of every host
    element type (src/lib/THClTensor.h:31-145, src/lib/THClStorageCopy.h:9-30)."""
    import ctypes as C
    from cltorch_amd.tensor import _call
    t = cl.ClTensor()
    _call("THClTensor_resize5d", t._h, 2, 1, 3, 1, 4)
    assert t.size() == (2, 1, 3, 1, 4) and t.isContiguous()
    u = cl.ClTensor()
    _call("THClTensor_squeeze1d", u._h, t._h, C.c_int(1))
    assert u.size() == (2, 3, 1, 4)
    _call("THClTensor_squeeze1d", u._h, u._h, C.c_int(0))            # size 2: nothing to drop
    assert u.size() == (2, 3, 1, 4)
    u.zero()
    _call("THClTensor_set4d", u._h, 1, 2, 0, 3, C.c_float(7.5))
    lib = cl.state().lib
    lib.THClTensor_get4d.restype = C.c_float
    assert _call("THClTensor_get4d", u._h, 1, 2, 0, 3) == 7.5 and u.float()[1, 2, 0, 3] == 7.5 and u.sum() == 7.5
    v = cl.ClTensor(3, 4, 5).zero().transpose(1, 3)
    _call("THClTensor_set3d", v._h, 4, 1, 2, C.c_float(-2.0))
    assert _call("THClTensor_get3d", v._h, 4, 1, 2) == -2.0 and v.float()[4, 1, 2] == -2.0
    with pytest.raises(cl.ClError):
        _call("THClTensor_get3d", v._h, 5, 0, 0)
    # whole storages
    a = cl.ClTensor(np.arange(10, dtype=F))
    b = cl.ClTensor(10).zero()
    sa = lib.THClTensor_storage(cl.state().ptr, a._h)
    sb = lib.THClTensor_storage(cl.state().ptr, b._h)
    _call("THClStorage_copy", sb, sa)
    assert b.float().tolist() == list(range(10))

    class _Storage(C.Structure):
        _fields_ = [("data", C.c_void_p), ("size", C.c_long), ("refcount", C.c_int), ("flag", C.c_char),
                    ("allocator", C.c_void_p), ("allocatorContext", C.c_void_p), ("view", C.c_void_p)]
    for name, dtype in (("Byte", np.uint8), ("Char", np.int8), ("Short", np.int16), ("Int", np.int32), ("Long", np.int64),
                        ("Double", np.float64)):
        h = (np.arange(10) * 3 % 100).astype(dtype)
        hs = _Storage(h.ctypes.data, 10, 1, b"\x00", None, None, None)
        _call(f"THClStorage_copy{name}", sb, C.byref(hs))
        assert b.float().tolist() == h.astype(F).tolist(), name
        out = np.zeros(10, dtype=dtype)
        os_ = _Storage(out.ctypes.data, 10, 1, b"\x00", None, None, None)
        _call(f"TH{name}Storage_copyCl", C.byref(os_), sa)
        assert out.tolist() == list(range(10)), name


def test_views_over_a_storage_with_sizes_spelled_out(cl):
    """newWithStorage1d..4d and setStorage1d..4d: sizes and strides as plain arguments, -1 for the
    dimensions that are not there and for strides to be derived (src/lib/THClTensor.cpp:136-171,342-386)."""
    import ctypes as C
    from cltorch_amd.tensor import _call
    lib, st = cl.state().lib, cl.state().ptr
    base = cl.ClTensor(np.arange(24, dtype=F))
    storage = C.c_void_p(lib.THClTensor_storage(st, base._h))
    L = C.c_long
    for name in ("THClTensor_newWithStorage1d", "THClTensor_newWithStorage2d", "THClTensor_newWithStorage3d", "THClTensor_newWithStorage4d"):
        getattr(lib, name).restype = C.c_void_p
    host = np.arange(24, dtype=F)

    def view(handle):
        t = cl.ClTensor()
        _call("THClTensor_set", t._h, C.c_void_p(handle))
        lib.THClTensor_free(st, C.c_void_p(handle))
        return t

    v1 = view(lib.THClTensor_newWithStorage1d(st, C.c_int(0), storage, L(2), L(5), L(4)))
    assert v1.size() == (5,) and v1.stride() == (4,) and v1.float().tolist() == host[2::4][:5].tolist()
    v2 = view(lib.THClTensor_newWithStorage2d(st, C.c_int(0), storage, L(0), L(4), L(6), L(6), L(1)))
    assert v2.size() == (4, 6) and np.array_equal(v2.float(), host.reshape(4, 6))
    v2t = view(lib.THClTensor_newWithStorage2d(st, C.c_int(0), storage, L(0), L(6), L(1), L(4), L(6)))
    assert np.array_equal(v2t.float(), host.reshape(4, 6).T)
    v3 = view(lib.THClTensor_newWithStorage3d(st, C.c_int(0), storage, L(0), L(2), L(-1), L(3), L(-1), L(4), L(-1)))
    assert v3.size() == (2, 3, 4) and v3.stride() == (12, 4, 1) and np.array_equal(v3.float(), host.reshape(2, 3, 4))
    v4 = view(lib.THClTensor_newWithStorage4d(st, C.c_int(0), storage, L(0), L(2), L(12), L(2), L(6), L(3), L(2), L(2), L(1)))
    assert v4.size() == (2, 2, 3, 2) and np.array_equal(v4.float(), host.reshape(2, 2, 3, 2))
    assert v4.sum() == float(host.sum())                      # kernels see the same elements
    t = cl.ClTensor()
    _call("THClTensor_setStorage1d", t._h, storage, L(20), L(4), L(1))
    assert t.float().tolist() == [20.0, 21.0, 22.0, 23.0]
    _call("THClTensor_setStorage2d", t._h, storage, L(1), L(3), L(8), L(2), L(3))
    assert np.array_equal(t.float(), np.array([[1, 4], [9, 12], [17, 20]], dtype=F))
    _call("THClTensor_setStorage3d", t._h, storage, L(0), L(2), L(12), L(2), L(6), L(6), L(1))
    assert np.array_equal(t.float(), host.reshape(2, 2, 6))
    _call("THClTensor_setStorage4d", t._h, storage, L(0), L(1), L(-1), L(2), L(-1), L(3), L(-1), L(4), L(-1))
    assert t.size() == (1, 2, 3, 4) and t.isContiguous()
    t.fill(-1.0)                                              # the view writes through to the shared storage
    assert base.float().tolist() == [-1.0] * 24
    with pytest.raises(cl.ClError):
        _call("THClTensor_setStorage1d", t._h, storage, L(-1), L(4), L(1))


def test_current_device_forms(cl):
    """The forms without a device argument act on the current device
    (src/lib/THClGeneral.cpp:119-133,178-185, src/lib/THClTensor.cpp:66-72,92-95,844-902,
    src/lib/THClStorage.cpp:93-96)."""
    import ctypes as C
    st = cl.state()
    lib, sp = st.lib, st.ptr
    cur = lib.THClState_getDevice(sp)
    ctx = lib.THClState_getClv2(sp, cur)
    assert lib.THClState_getCl(sp) == ctx
    dev = C.c_int(-5)
    assert lib.THClState_getClAndDevice(sp, C.byref(dev)) == ctx and dev.value == cur
    assert lib.THClState_getClAndDevice(sp, None) == ctx
    assert lib.THClState_getCurrentDeviceScratchSpace(sp) == lib.THClState_getDeviceScratchSpace(sp, cur, 0)
    assert lib.THClState_getCurrentDeviceScratchSpaceSize(sp) == lib.THClState_getDeviceScratchSpaceSize(sp, cur) > 0
    t = lib.THClTensor_new(sp)
    s = lib.THClStorage_new(sp)
    assert lib.THClTensor_getDevice(sp, t) == cur and lib.THClStorage_size(sp, s) == 0
    assert lib.THClTensor_wrapper(sp, t) is None and lib.THClTensor_getCl(sp, t) is None
    a = cl.ClTensor(np.arange(6, dtype=F)).narrow(1, 3, 2)
    assert lib.THClTensor_getCl(sp, a._h) == ctx
    base = lib.THClTensor_wrapper(sp, a._h)
    assert lib.THClTensor_data(sp, a._h) == base + 2 * 4
    assert lib.THClTensor_checkGPU(sp, C.c_uint(3), C.c_void_p(a._h), C.c_void_p(None), C.c_void_p(t)) == 1
    assert lib.THClTensor_checkGPU(sp, C.c_uint(0)) == 1
    lib.THClTensor_free(sp, t)
    lib.THClStorage_free(sp, s)


def test_save_and_load(cl, tmp_path):
    """torch.save / torch.load of a ClTensor (src/test/unit_tensor.lua:1033-1052: values with NaN
    and infinities come back as they were), and a strided view keeps its sizes, strides and offset."""
    a = cl.ClTensor(np.array([3, 5, 4.7, np.nan, np.inf], dtype=F))
    path = str(tmp_path / "out.dat")
    cl.save(path, a)
    b = cl.load(path)
    assert b.size() == a.size()
    assert np.array_equal(a.float().view(np.uint32), b.float().view(np.uint32))
    base = cl.ClTensor(np.arange(60, dtype=F).reshape(3, 4, 5))
    v = base.transpose(1, 3).narrow(2, 2, 2)
    cl.save(path, v)
    w = cl.load(path)
    assert (w.size(), w.stride(), w.storageOffset()) == (v.size(), v.stride(), v.storageOffset())
    assert np.array_equal(w.float(), v.float())
    cl.save(path, cl.ClTensor())
    e = cl.load(path)
    assert e.nElement() == 0 and e.nDimension() == cl.ClTensor().nDimension()
    # a point tensor keeps its value (and stays a point tensor); NaN and infinities included
    for value in (2.5, float("inf"), float("nan")):
        src = cl.ClTensor(np.array([1.0, value], dtype=F))
        p = cl.ClTensor()
        p.sum(src.narrow(1, 2, 1))
        assert p.nDimension() == 0
        cl.save(path, p)
        q = cl.load(path)
        assert q.nDimension() == 0
        assert np.array([q.s()], dtype=F).view(np.uint32)[0] == np.array([value], dtype=F).view(np.uint32)[0] or (value != value and q.s() != q.s())
    # an empty header as the reference itself would write it (dimension count -1, no storage)
    import struct
    from cltorch_amd import serialize
    raw = serialize.encode_tensor([], [], 0, None)
    at = raw.index(b"torch.ClTensor") + len(b"torch.ClTensor")
    assert raw[at:at + 4] == struct.pack("=i", -1)
    with open(path, "wb") as f:
        f.write(raw)
    assert cl.load(path).nElement() == 0
    with open(path, "wb") as f:          # a writer that puts 0 there reads back as empty as well
        f.write(raw[:at] + struct.pack("=i", 0) + raw[at + 4:])
    assert cl.load(path).nElement() == 0
    cl.save(path, cl.ClTensor())
    assert open(path, "rb").read() == raw
