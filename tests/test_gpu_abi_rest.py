"""Entry points of the C ABI that the ctypes mirror does not route through: the in-place view forms, the sized
constructors and resizes, flags, the remaining point-tensor operators and copies.  Each is called by its exported
name and checked against numpy on the same data."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F = np.float32


def _longs(cl, st):
    """values of a host THLongStorage (freed here)"""
    from cltorch_amd.tensor import _LongStorageStruct
    s = C.cast(st, C.POINTER(_LongStorageStruct)).contents
    out = [int(s.data[i]) for i in range(s.size)]
    cl.state().lib.THLongStorage_free(st)
    return out


def test_views_made_in_place(cl):
    """narrow / select / transpose / unfold turn `self` into a view of `src`, or of itself when src is NULL
    (src/lib/THClTensor.cpp:389-500)."""
    from cltorch_amd.tensor import _call
    a = np.arange(4 * 5 * 6, dtype=F).reshape(4, 5, 6)
    A = cl.ClTensor(a)
    V = cl.ClTensor()
    _call("THClTensor_narrow", V._h, A._h, 1, 1, 3)
    assert V.size() == (4, 3, 6) and np.array_equal(V.float(), a[:, 1:4])
    _call("THClTensor_narrow", V._h, None, 2, 2, 2)        # of itself
    assert np.array_equal(V.float(), a[:, 1:4, 2:4])
    _call("THClTensor_select", V._h, A._h, 0, 2)
    assert V.size() == (5, 6) and np.array_equal(V.float(), a[2])
    _call("THClTensor_transpose", V._h, A._h, 0, 2)
    assert V.size() == (6, 5, 4) and np.array_equal(V.float(), a.transpose(2, 1, 0))
    _call("THClTensor_transpose", V._h, None, 0, 1)
    assert np.array_equal(V.float(), a.transpose(1, 2, 0))
    _call("THClTensor_unfold", V._h, A._h, 2, 3, 2)          # windows of 3, step 2, along the last dim
    assert V.size() == (4, 5, 2, 3)
    want = np.stack([a[:, :, 0:3], a[:, :, 2:5]], axis=2)
    assert np.array_equal(V.float(), want)
    # the view shares A's storage: a write through it shows in A
    V.fill(-1.0)
    a2 = a.copy()
    a2[:, :, 0:5] = -1.0
    assert np.array_equal(A.float(), a2)
    # a select of the only dimension is refused, as in the reference
    one = cl.ClTensor(np.arange(3, dtype=F))
    with pytest.raises(cl.ClError):
        _call("THClTensor_select", V._h, one._h, 0, 1)


def test_sized_constructors_resizes_and_metadata(cl):
    """newWithSize1d..4d, resize0d/1d/3d/4d, newSizeOf / newStrideOf, numel, isSameSizeAs
    (src/lib/THClTensor.cpp:45-58, 178-200, 287-326, 567-580; src/lib/THClTensorMath.cpp:106-109)."""
    from cltorch_amd.tensor import _call
    for sizes in ((7,), (3, 5), (2, 3, 4), (2, 3, 4, 5)):
        h = _call("THClTensor_newWithSize%dd" % len(sizes), 0, *[C.c_long(s) for s in sizes])
        t = cl.ClTensor(_handle=h)
        assert t.size() == sizes and t.isContiguous()
        assert _longs(cl, _call("THClTensor_newSizeOf", h)) == list(sizes)
        strides = [int(np.prod(sizes[i + 1:])) for i in range(len(sizes))]
        assert _longs(cl, _call("THClTensor_newStrideOf", h)) == strides
        assert _call("THClTensor_numel", h) == int(np.prod(sizes))
        t.fill(2.0)
        assert float(t.sum()) == 2.0 * np.prod(sizes)
    t = cl.ClTensor(6)
    t.copy(cl.ClTensor(np.arange(6, dtype=F)))
    u = cl.ClTensor(2, 3)
    assert not _call("THClTensor_isSameSizeAs", t._h, u._h)
    _call("THClTensor_resize3d", t._h, C.c_long(1), C.c_long(2), C.c_long(3))
    assert t.size() == (1, 2, 3) and np.array_equal(t.float().ravel(), np.arange(6, dtype=F))   # same storage, no copy
    _call("THClTensor_resize4d", t._h, C.c_long(1), C.c_long(3), C.c_long(1), C.c_long(2))
    assert t.size() == (1, 3, 1, 2)
    _call("THClTensor_resize1d", t._h, C.c_long(4))
    assert t.size() == (4,) and np.array_equal(t.float(), np.arange(4, dtype=F))
    _call("THClTensor_resize1d", u._h, C.c_long(4))
    assert _call("THClTensor_isSameSizeAs", t._h, u._h)
    _call("THClTensor_resize0d", t._h)
    assert t.nDimension() == 0


def test_zeros_ones_and_set_storage(cl):
    """zeros / ones resize and fill (src/lib/THClTensorMath.cpp:83-104); setStorage points a header at a storage
    with an offset, sizes and strides of the caller's choosing (src/lib/THClTensor.cpp:328-345)."""
    from cltorch_amd.tensor import _call, _long_storage
    lib = cl.state().lib
    t = cl.ClTensor(np.full((5,), 9.0, F))
    sz = _long_storage([3, 4])
    _call("THClTensor_zeros", t._h, sz)
    assert t.size() == (3, 4) and np.array_equal(t.float(), np.zeros((3, 4), F))
    _call("THClTensor_ones", t._h, sz)
    assert np.array_equal(t.float(), np.ones((3, 4), F))
    lib.THLongStorage_free(sz)

    st = cl.ClStorage(np.arange(24, dtype=F))
    v = cl.ClTensor()
    sz, sd = _long_storage([3, 2]), _long_storage([2, 7])
    _call("THClTensor_setStorage", v._h, st._h, C.c_long(5), sz, sd)
    lib.THLongStorage_free(sz)
    lib.THLongStorage_free(sd)
    want = np.array([[5 + 2 * i + 7 * j for j in range(2)] for i in range(3)], F)
    assert v.size() == (3, 2) and v.stride() == (2, 7) and v.storageOffset() == 6
    assert np.array_equal(v.float(), want)
    v.mul(2.0)          # through the view into the storage
    host = st.to_host()
    base = np.arange(24, dtype=F)
    base[want.astype(int).ravel()] *= 2
    assert np.array_equal(host, base)


def test_flags_and_reference_counts(cl):
    """A header or storage whose REFCOUNTED flag is cleared is neither retained nor freed; with the flag back
    it counts again, and a retained storage outlives the header that made it
    (src/lib/THClTensor.cpp:74-84, 590-616; src/lib/THClStorage.cpp:202-223)."""
    from cltorch_amd.tensor import _call
    REFCOUNTED = C.c_char(bytes([1]))

    class Head(C.Structure):     # leading fields of THClTensor
        _fields_ = [("size", C.c_void_p), ("stride", C.c_void_p), ("nDimension", C.c_int), ("storage", C.c_void_p),
                    ("storageOffset", C.c_long), ("refcount", C.c_int), ("flag", C.c_char)]

    class Store(C.Structure):    # leading fields of THClStorage
        _fields_ = [("device", C.c_int), ("data", C.c_void_p), ("cl", C.c_void_p), ("wrapper", C.c_void_p),
                    ("size", C.c_long), ("refcount", C.c_int), ("flag", C.c_char)]
    t = cl.ClTensor(np.arange(8, dtype=F))
    head = C.cast(t._h, C.POINTER(Head)).contents
    assert head.refcount == 1 and head.flag[0] & 1
    _call("THClTensor_clearFlag", t._h, REFCOUNTED)
    assert not head.flag[0] & 1
    _call("THClTensor_retain", t._h)
    assert head.refcount == 1
    _call("THClTensor_free", t._h)                   # no effect either: the header is still there
    assert head.refcount == 1 and t.size() == (8,)
    _call("THClTensor_setFlag", t._h, REFCOUNTED)
    _call("THClTensor_retain", t._h)
    assert head.refcount == 2
    _call("THClTensor_free", t._h)
    assert head.refcount == 1

    st = _call("THClTensor_storage", t._h)
    store = C.cast(st, C.POINTER(Store)).contents
    assert store.refcount == 1 and store.size == 8
    _call("THClStorage_clearFlag", st, REFCOUNTED)
    _call("THClStorage_retain", st)
    assert store.refcount == 1
    _call("THClStorage_setFlag", st, REFCOUNTED)
    _call("THClStorage_retain", st)
    assert store.refcount == 2
    del t                                            # the header goes, the storage stays for its second owner
    assert store.refcount == 1
    keep = cl.ClStorage.__new__(cl.ClStorage)
    keep._lib, keep._h = cl.state().lib, st
    assert np.array_equal(keep.to_host(), np.arange(8, dtype=F))
    assert _call("THClStorage_data", st) is None     # no host mirror unless a caller asked for one


def test_point_tensor_add_sub_and_product(cl):
    """add_gpu / sub_gpu take their scalar from a point tensor on the device, prodall_gpu leaves the product
    in one (src/lib/THClTensorMathPairwise.cpp:155-187, src/lib/THClTensorMath.cpp:408-411)."""
    from cltorch_amd.tensor import _call
    rng = np.random.RandomState(3)
    for n in (1, 5, 1000, (1 << 20) + 3):
        a = rng.uniform(0.5, 1.5, n).astype(F)
        A = cl.ClTensor(a)
        pt = cl.ClTensor()
        _call("THClTensor_sumall_gpu", pt._h, A._h)
        s = F(pt.s())
        R = cl.ClTensor()
        _call("THClTensor_add_gpu", R._h, A._h, pt._h)
        assert np.array_equal(R.float(), a + s)
        _call("THClTensor_sub_gpu", A._h, A._h, pt._h)          # in place
        assert np.array_equal(A.float(), a - s)
    # product: exact while every partial product is a small integer or power of two
    v = np.array([2, 0.5, 4, 0.25, 3, 2, 0.5, 1, 1, 8] * 7, F)
    P = cl.ClTensor(v)
    pt = cl.ClTensor()
    _call("THClTensor_prodall_gpu", pt._h, P._h)
    assert pt.s() == float(np.prod(v.astype(np.float64)))
    assert pt.nDimension() == 0          # a point tensor: no dimensions, one element of storage


def test_device_and_long_copies(cl):
    """copyCl is the device-to-device copy under its generic name, copyLong takes a host LongTensor of any layout,
    freeCopyTo hands a temporary's values to its destination and drops it
    (src/lib/THClTensorCopy.cpp:38-66, 130-230; src/lib/THClTensor.cpp:618-624)."""
    from cltorch_amd.tensor import _call, _long_vector
    lib = cl.state().lib
    a = np.arange(30, dtype=F).reshape(5, 6)
    A = cl.ClTensor(a)
    B = cl.ClTensor(6, 5)
    At = A.t()
    _call("THClTensor_copyCl", B._h, At._h)
    assert np.array_equal(B.float(), a.T)

    lt = _long_vector(np.arange(30, dtype=np.int64) * 3 - 7)
    D = cl.ClTensor(5, 6)
    _call("THClTensor_copyLong", D._h, lt)
    lib.THLongTensor_free(lt)
    assert np.array_equal(D.float(), (np.arange(30) * 3 - 7).astype(F).reshape(5, 6))
    short = _long_vector([1, 2, 3])
    with pytest.raises(cl.ClError):
        _call("THClTensor_copyLong", D._h, short)
    lib.THLongTensor_free(short)

    tmp = _call("THClTensor_newClone", A._h)
    cl.ClTensor(_handle=_call("THClTensor_newNarrow", tmp, 0, 0, 5)).mul(2.0)     # a second header, gone right away
    dst = cl.ClTensor(5, 6)
    _call("THClTensor_freeCopyTo", tmp, dst._h)                                   # tmp is freed by the call
    assert np.array_equal(dst.float(), a * 2)


def test_storage_raw_copy_and_kernel_argument_count(cl):
    """rawCopy fills a storage from a bare host pointer (src/lib/THClStorageCopy.cpp:11-20); a user kernel
    reports how many arguments it was declared with (src/UserKernel.cpp:217-300)."""
    from cltorch_amd.tensor import _call
    st = cl.ClStorage(12)
    src = np.arange(12, dtype=F) * 0.5
    _call("THClStorage_rawCopy", st._h, src.ctypes.data_as(C.POINTER(C.c_float)))
    assert np.array_equal(st.to_host(), src)
    assert _call("THClStorage_size", st._h) == 12

    k = cl.ClKernel({"input": {"nElements": "int", "scale": "float", "src": "ClTensor"}, "output": {"dst": "ClTensor"},
                     "src": "int i = get_global_id(0); if (i < nElements) dst_data[i] = scale * src_data[i];"})
    assert cl.state().lib.THClKernel_numArgs(k._h) == 4
    cl.state().lib.THClSetAllowNonGpus(cl.state().ptr, 1)       # accepted and without effect: there is no non-GPU device
    x = cl.ClTensor(np.arange(10, dtype=F))
    y = cl.ClTensor(10)
    k.run({"nElements": 10, "scale": 3.0, "src": x, "dst": y})
    assert np.array_equal(y.float(), np.arange(10, dtype=F) * 3)
