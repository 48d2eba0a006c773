"""Host-side mirror of cltorch's Lua ``torch.ClTensor`` for the hot path.

The reference's user-facing layer is Lua (``src/TensorMath.lua`` declares every
method and overload; cwrap turns them into calls of ``THClTensor_*``).  Lua is
not available here, so this module plays the role of that generated layer over
the same C ABI: same method names, same overload resolution
(``src/TensorMath.lua:655-668,727-736,943-988``), **1-based dimensions and
1-based returned indices** as in Lua, results returned the way the Lua methods
return them.  All arithmetic happens in ``libthcl_hip.so``; nothing here
computes on the host.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple, Union

import numpy as np

from . import _lib


class ClError(RuntimeError):
    """A check inside the library failed (what Torch7 raises as a Lua error)."""


class _State:
    """The global THClState that ``require 'cltorch'`` creates (``src/init.cpp:229-249``)."""

    def __init__(self):
        self.lib = _lib.load()
        self.buf = C.create_string_buffer(256)  # larger than sizeof(THClState)
        self.ptr = C.cast(self.buf, C.c_void_p)
        self.lib.THCl_initializeState(self.ptr)
        self.lib.THClInit(self.ptr)
        err = self.lib.THClLastError()
        if err:
            raise ClError(err.decode())

    def check(self):
        err = self.lib.THClLastError()
        if err:
            msg = err.decode()
            self.lib.THClClearError()
            raise ClError(msg)


_state: Optional[_State] = None


def state() -> _State:
    global _state
    if _state is None:
        _state = _State()
    return _state


def _call(name: str, *args):
    st = state()
    r = getattr(st.lib, name)(st.ptr, *args)
    st.check()
    return r


def synchronize() -> None:
    """``cltorch.synchronize()`` / ``cltorch.finish()``."""
    _call("THClState_synchronize")


finish = synchronize


def memoryStats(device: int = 1) -> dict:
    """Bytes in live tensors, bytes kept in the block cache, and how many requests
    went to the driver or were served from the cache (device is 1-based)."""
    st = state()
    rt = st.lib.THClState_getClv2(st.ptr, device - 1)
    live, cached = C.c_size_t(0), C.c_size_t(0)
    mallocs, hits = C.c_ulonglong(0), C.c_ulonglong(0)
    st.lib.thcl_rt_memory_stats(rt, C.byref(live), C.byref(cached), C.byref(mallocs), C.byref(hits))
    return {"live_bytes": live.value, "cached_bytes": cached.value, "device_mallocs": mallocs.value, "cache_hits": hits.value}


def emptyCache(device: int = 1) -> None:
    """Hands every cached block back to the driver."""
    st = state()
    st.lib.thcl_rt_empty_cache(st.lib.THClState_getClv2(st.ptr, device - 1))


def setProfiling(on) -> None:
    """``cltorch.setProfiling(1)``: time every launch with device events."""
    _call("THClState_setProfiling", C.c_int(1 if on else 0))


def dumpProfiling() -> str:
    """``cltorch.dumpProfiling()``: per entry point -- launches, total and mean ms; clears the records."""
    buf = C.create_string_buffer(1 << 16)
    _call("THClState_dumpProfiling", buf, C.c_long(len(buf)))
    return buf.value.decode()


def getDeviceCount() -> int:
    return int(_call("THClState_getNumDevices"))


def setAddFinish(flag: int) -> None:
    _state_int(5, flag)


class _PinnedOwner:
    def __init__(self, lib, ptr):
        self.lib, self.ptr = lib, ptr

    def __del__(self):
        try:
            if self.ptr and self.lib is not None:
                self.lib.thcl_rt_host_free(self.ptr)
                self.ptr = None
        except Exception:
            pass


def pinned_array(shape, dtype=np.float32) -> np.ndarray:
    """A numpy array in page-locked host memory: copies between it and a ClTensor run at the link's
    rate instead of the pageable-memory rate.  The memory is released with the array."""
    st = state()
    getDeviceCount()                                  # initialises the runtime
    count = int(np.prod(shape)) if np.ndim(shape) else int(shape)
    nbytes = max(count, 1) * np.dtype(dtype).itemsize
    fn = st.lib.thcl_rt_host_alloc
    fn.restype = C.c_void_p
    ptr = fn(C.c_size_t(nbytes))
    if not ptr:
        raise ClError("pinned allocation failed: " + st.lib.thcl_rt_error().decode())
    owner = _PinnedOwner(st.lib, ptr)
    buf = (C.c_char * nbytes).from_address(ptr)
    buf._owner = owner                                # keeps the allocation alive as long as any view of it
    return np.frombuffer(buf, dtype=dtype, count=count).reshape(shape)


def getDevice() -> int:
    """``cltorch.getDevice()`` (1-based, src/init.cpp:44-50)."""
    return int(_call("THClState_getDevice")) + 1


def setDevice(device: int) -> None:
    """``cltorch.setDevice(device)`` (1-based, src/init.cpp:52-59)."""
    _call("THClState_setDevice", C.c_int(device - 1))


class _RtProps(C.Structure):  # thcl_rt_props of include/thcl_rt.h
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int), ("wavefront", C.c_int),
                ("max_threads_per_block", C.c_int), ("clock_khz", C.c_int), ("lds_bytes_per_block", C.c_int),
                ("total_mem", C.c_size_t)]


def getDeviceProperties(device: int) -> dict:
    """``cltorch.getDeviceProperties(device)``: the reference's keys (src/init.cpp:79-121) where HIP has a
    counterpart, plus the code-object architecture and the wavefront width."""
    st = state()
    if device < 1 or device > getDeviceCount():
        raise ClError("Device doesnt exist")
    fn = st.lib.thcl_rt_get_props
    fn.restype = C.POINTER(_RtProps)
    p = fn(st.lib.THClState_getClv2(st.ptr, device - 1)).contents
    st.check()
    return {"deviceName": p.name.decode(), "deviceType": "GPU", "platformVendor": "Advanced Micro Devices, Inc.",
            "maxComputeUnits": p.compute_units, "maxWorkGroupSize": p.max_threads_per_block,
            "maxClockFrequency": p.clock_khz // 1000, "globalMemSizeMB": p.total_mem // (1 << 20),
            "maxMemAllocSizeMB": p.total_mem // (1 << 20), "localMemSizeKB": p.lds_bytes_per_block // 1024,
            "deviceVersion": p.arch.decode(), "wavefrontSize": p.wavefront}


def _state_int(index: int, value: int) -> None:
    # THClState starts with ints: initialized, allowNonGpus, allocatedDevices, currentDevice, trace, addFinish,
    # detailedTimings (include/thcl_hip.h, field order of src/lib/THClGeneral.h:76-93)
    C.cast(state().buf, C.POINTER(C.c_int))[index] = int(value)


def setTrace(flag: int) -> None:
    """``cltorch.setTrace(1)`` (src/init.cpp:61-67): the state's trace flag."""
    _state_int(4, flag)


def setDetailedTimings(flag: int) -> None:
    _state_int(6, flag)


def setEnableTiming(flag) -> None:
    """``cltorch.setEnableTiming`` / ``setTiming``: the reference's host-side timers map onto launch profiling."""
    setProfiling(flag)


setTiming = setEnableTiming


def dumpTimings() -> str:
    """``cltorch.dumpTimings()``: same records as :func:`dumpProfiling`."""
    return dumpProfiling()


def about() -> str:
    """``cltorch.about()`` (src/init.cpp:180-196)."""
    return "cltorch_amd: cltorch's tensor operator API on AMD Instinct GPUs through HIP\n"


_rng = np.random.RandomState(5489)


def manualSeed(seed: int) -> None:
    """``torch.manualSeed(seed)`` for the host-side generator behind ``uniform`` / ``bernoulli`` / ``normal``."""
    global _rng
    _rng = np.random.RandomState(int(seed) & 0xFFFFFFFF)


def _uniform01(n: int) -> np.ndarray:
    # one 32-bit Mersenne-Twister word per value, scaled by 2^-32 (Torch7's THRandom_uniform)
    return _rng.randint(0, 1 << 32, size=n, dtype=np.uint64).astype(np.float64) * (1.0 / 4294967296.0)


def _long_storage(values: Sequence[int]):
    lib = state().lib
    s = lib.THLongStorage_newWithSize(len(values))
    for i, v in enumerate(values):
        lib.THLongStorage_set(s, i, int(v))
    return s


class _LongStorageStruct(C.Structure):
    _fields_ = [("data", C.POINTER(C.c_long)), ("size", C.c_long)]


class _LongTensorStruct(C.Structure):  # THLongTensor: size*, stride*, int nDimension, storage*
    _fields_ = [("size", C.c_void_p), ("stride", C.c_void_p), ("nDimension", C.c_int),
                ("storage", C.POINTER(_LongStorageStruct))]


def _long_vector(values):
    """A host ``torch.LongTensor`` vector holding ``values``; the caller frees it."""
    lib = state().lib
    vals = np.asarray(values, dtype=np.int64).reshape(-1)
    sz = _long_storage([vals.size])
    lt = lib.THLongTensor_newWithSize(sz, None)
    lib.THLongStorage_free(sz)
    if vals.size:
        t = C.cast(lt, C.POINTER(_LongTensorStruct)).contents
        np.ctypeslib.as_array(t.storage.contents.data, shape=(vals.size,))[:] = vals
    return lt


class ClTensor:
    """``torch.ClTensor``: a strided fp32 view of device storage."""

    def __init__(self, *sizes, _handle=None, device: int = 0):
        self._lib = state().lib
        if _handle is not None:
            self._h = _handle
            return
        if len(sizes) == 1 and isinstance(sizes[0], (list, tuple, np.ndarray)) and not isinstance(sizes[0], (int,)):
            arr = np.asarray(sizes[0], dtype=np.float32)
            self._h = _call("THClTensor_newv2", device)
            self._resize(arr.shape)
            self._upload(arr)
            return
        self._h = _call("THClTensor_newv2", device)
        if sizes:
            self._resize(sizes)

    # ---- lifecycle ------------------------------------------------------
    def __del__(self):
        try:
            if getattr(self, "_h", None) and _state is not None:
                self._lib.THClTensor_free(_state.ptr, self._h)
                self._h = None
        except Exception:
            pass

    def _resize(self, sizes):
        s = _long_storage(list(sizes))
        try:
            _call("THClTensor_resize", self._h, s, None)
        finally:
            self._lib.THLongStorage_free(s)

    def _upload(self, arr: np.ndarray):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        sz = (C.c_long * max(arr.ndim, 1))(*arr.shape)
        ft = self._lib.THFloatTensor_newWithData(arr.ctypes.data_as(C.c_void_p), arr.size, 0, arr.ndim, sz, None)
        try:
            _call("THClTensor_copyFloat", self._h, ft)
        finally:
            self._lib.THFloatTensor_free(ft)

    @staticmethod
    def from_numpy(arr) -> "ClTensor":
        """``floatTensor:cl()``"""
        return ClTensor(np.asarray(arr, dtype=np.float32))

    # ---- metadata ---------------------------------------------------------
    def nDimension(self) -> int:
        return int(_call("THClTensor_nDimension", self._h))

    dim = nDimension

    def size(self, dim: Optional[int] = None):
        nd = max(self.nDimension(), 0)
        if dim is not None:
            return int(_call("THClTensor_size", self._h, dim - 1))
        return tuple(int(_call("THClTensor_size", self._h, d)) for d in range(nd))

    def stride(self, dim: Optional[int] = None):
        nd = max(self.nDimension(), 0)
        if dim is not None:
            return int(_call("THClTensor_stride", self._h, dim - 1))
        return tuple(int(_call("THClTensor_stride", self._h, d)) for d in range(nd))

    def storageOffset(self) -> int:
        """1-based, as in Lua."""
        return int(_call("THClTensor_storageOffset", self._h)) + 1

    def nElement(self) -> int:
        return int(_call("THClTensor_nElement", self._h))

    numel = nElement

    def isContiguous(self) -> bool:
        return bool(_call("THClTensor_isContiguous", self._h))

    def data_ptr(self) -> int:
        return int(_call("THClTensor_data", self._h) or 0)

    # ---- views (header only) ---------------------------------------------
    def _wrap(self, h) -> "ClTensor":
        if not h:
            state().check()
            raise ClError("view creation failed")
        return ClTensor(_handle=h)

    def narrow(self, dim: int, first: int, size: int) -> "ClTensor":
        return self._wrap(_call("THClTensor_newNarrow", self._h, dim - 1, first - 1, size))

    def select(self, dim: int, index: int) -> "ClTensor":
        return self._wrap(_call("THClTensor_newSelect", self._h, dim - 1, index - 1))

    def transpose(self, d1: int, d2: int) -> "ClTensor":
        return self._wrap(_call("THClTensor_newTranspose", self._h, d1 - 1, d2 - 1))

    def t(self) -> "ClTensor":
        if self.nDimension() != 2:
            raise ClError("t() expects a 2D tensor")
        return self.transpose(1, 2)

    def unfold(self, dim: int, size: int, step: int) -> "ClTensor":
        return self._wrap(_call("THClTensor_newUnfold", self._h, dim - 1, size, step))

    def strided(self, sizes: Sequence[int], strides: Sequence[int], offset: int = 1) -> "ClTensor":
        """View of the same storage with explicit sizes/strides (``torch.ClTensor(storage, offset, sizes, strides)``)."""
        st = _call("THClTensor_storage", self._h)
        sz, sd = _long_storage(sizes), _long_storage(strides)
        try:
            h = _call("THClTensor_newWithStorage", 0, st, offset - 1, sz, sd)
        finally:
            self._lib.THLongStorage_free(sz)
            self._lib.THLongStorage_free(sd)
        return self._wrap(h)

    # ---- header-only views the Lua binding borrows from torch (src/Tensor.lua:74-81) --------
    def _view_of(self, sizes, strides) -> "ClTensor":
        return self.strided(list(sizes), list(strides), self.storageOffset())

    def sub(self, *bounds) -> "ClTensor":
        """``a:sub(i1, j1 [, i2, j2 ...])``: a narrow per leading dim; negative bounds count from the end."""
        t = self
        for d in range(0, len(bounds), 2):
            n = t.size(d // 2 + 1)
            lo, hi = bounds[d], bounds[d + 1]
            lo = lo + n + 1 if lo < 0 else lo
            hi = hi + n + 1 if hi < 0 else hi
            if not (1 <= lo <= hi <= n):
                raise ClError("sub: index out of range")
            t = t.narrow(d // 2 + 1, lo, hi - lo + 1)
        return t

    def expand(self, *sizes) -> "ClTensor":
        """``a:expand(s1, s2, ...)``: dims of size 1 repeat with stride 0; the other sizes must match."""
        sizes = list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes)
        have, st = self.size(), self.stride()
        if len(sizes) != len(have):
            raise ClError("the number of dimensions provided must equal tensor:dim()")
        strides = []
        for d, (want, got) in enumerate(zip(sizes, have)):
            if got == 1:
                strides.append(0 if want != 1 else st[d])
            elif want == got:
                strides.append(st[d])
            else:
                raise ClError("incorrect size: only supporting singleton expansion (size=1)")
        return self._view_of(sizes, strides)

    def expandAs(self, other: "ClTensor") -> "ClTensor":
        return self.expand(*other.size())

    def view(self, *sizes) -> "ClTensor":
        """``a:view(s1, s2, ...)`` of a contiguous tensor; one size may be -1."""
        sizes = list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes)
        if not self.isContiguous():
            raise ClError("expecting a contiguous tensor")
        n = self.nElement()
        if sizes.count(-1) > 1:
            raise ClError("only one dimension can be at -1")
        if -1 in sizes:
            rest = int(np.prod([x for x in sizes if x != -1]))
            if rest == 0 or n % rest:
                raise ClError("input view size not compatible with input tensor size")
            sizes[sizes.index(-1)] = n // rest
        if int(np.prod(sizes)) != n:
            raise ClError("Wrong size for view. Input size: %d. Output size: %s" % (n, "x".join(map(str, sizes))))
        strides = [1] * len(sizes)
        for d in range(len(sizes) - 2, -1, -1):
            strides[d] = strides[d + 1] * sizes[d + 1]
        return self._view_of(sizes, strides)

    def viewAs(self, other: "ClTensor") -> "ClTensor":
        return self.view(*other.size())

    def permute(self, *order) -> "ClTensor":
        """``a:permute(d1, d2, ...)``: dim i of the result is dim ``order[i]`` of a."""
        nd = self.nDimension()
        if sorted(order) != list(range(1, nd + 1)):
            raise ClError("Invalid permutation")
        sz, st = self.size(), self.stride()
        return self._view_of([sz[o - 1] for o in order], [st[o - 1] for o in order])

    def split(self, size: int, dim: int = 1):
        """``a:split(size, dim)``: narrow views of at most ``size`` along dim."""
        n = self.size(dim)
        return [self.narrow(dim, lo, min(size, n - lo + 1)) for lo in range(1, n + 1, size)]

    def chunk(self, parts: int, dim: int = 1):
        return self.split(-(-self.size(dim) // parts), dim)

    def repeatTensor(self, *sizes) -> "ClTensor":
        """``a:repeatTensor(r1, r2, ...)``: a new tensor tiling a; built as torch does, by unfolding the
        result into blocks of a's shape and copying an expanded view of a into them."""
        sizes = list(sizes[0]) if len(sizes) == 1 and isinstance(sizes[0], (list, tuple)) else list(sizes)
        if len(sizes) < self.nDimension():
            raise ClError("Number of dimensions of repeat dims can not be smaller than number of dimensions of tensor")
        src = self.contiguous()
        xsize = [1] * (len(sizes) - self.nDimension()) + list(self.size())
        x = src.view(*xsize)
        result = ClTensor(*[a * b for a, b in zip(xsize, sizes)])
        blocks = result
        for d, s in enumerate(xsize):
            blocks = blocks.unfold(d + 1, s, s)
        x = x.view(*([1] * len(xsize) + xsize))
        blocks.copy(x.expandAs(blocks))
        return result

    # ---- Lua indexing (src/torch/generic/Tensor.cpp:782-1148) -----------------------------
    def __getitem__(self, key):
        """``a[i]``: the number at i of a vector, else ``select(1, i)``; ``a[mask]``: ``maskedSelect``;
        ``a[{i, {lo, hi}, ...}]`` as a tuple of ints and (lo, hi) pairs: select / narrow per dim."""
        if isinstance(key, ClTensor):
            return self.maskedSelect(key)
        if isinstance(key, (int, np.integer)):
            key = int(key) + self.size(1) + 1 if key < 0 else int(key)
            if self.nDimension() == 1:
                return float(_call("THClTensor_get1d", self._h, key - 1))
            return self.select(1, key)
        return self._index_view(key)

    def _index_view(self, key) -> "ClTensor":
        t, d = self, 1
        for k in key:
            if isinstance(k, (int, np.integer)):
                k = int(k) + t.size(d) + 1 if k < 0 else int(k)
                if t.nDimension() > 1:
                    t = t.select(d, k)          # the dim goes away, d now names the next one
                else:
                    t = t.narrow(1, k, 1)
                    d += 1
            else:
                k = tuple(k)                    # (): the whole dim, (i,): i alone with the dim kept, (lo, hi): a range
                n = t.size(d)
                lo = k[0] if len(k) > 0 else 1
                hi = k[1] if len(k) > 1 else (lo if len(k) == 1 else n)
                lo = lo + n + 1 if lo < 0 else lo
                hi = hi + n + 1 if hi < 0 else hi
                t = t.narrow(d, lo, hi - lo + 1)
                d += 1
        return t

    def __setitem__(self, key, value) -> None:
        """``a[i] = v``, ``a[mask] = v`` (``maskedFill``), ``a[{...}] = number or tensor``."""
        if isinstance(key, ClTensor):
            if isinstance(value, ClTensor):
                self.maskedCopy(key, value)
            else:
                self.maskedFill(key, value)
            return
        if isinstance(key, (int, np.integer)) and self.nDimension() == 1 and not isinstance(value, ClTensor):
            key = int(key) + self.size(1) + 1 if key < 0 else int(key)
            _call("THClTensor_set1d", self._h, key - 1, C.c_float(value))
            return
        view = self[key] if not isinstance(key, (int, np.integer)) else self.select(1, int(key) + self.size(1) + 1 if key < 0 else int(key))
        if isinstance(value, ClTensor):
            view.copy(value)
        else:
            view.fill(value)

    def reshape(self, *sizes) -> "ClTensor":
        """``a:reshape(s1, s2, ...)``: a new dense tensor with a's elements in order (``torch.reshape``)."""
        res = ClTensor()
        sz = _long_storage(list(sizes[0]) if len(sizes) == 1 and not isinstance(sizes[0], int) else list(sizes))
        try:
            _call("THClTensor_reshape", res._h, self._h, sz)
        finally:
            self._lib.THLongStorage_free(sz)
        return res

    def clone(self) -> "ClTensor":
        return self._wrap(_call("THClTensor_newClone", self._h))

    def contiguous(self) -> "ClTensor":
        return self._wrap(_call("THClTensor_newContiguous", self._h))

    def resize(self, *sizes) -> "ClTensor":
        self._resize(sizes)
        return self

    def resizeAs(self, other: "ClTensor") -> "ClTensor":
        _call("THClTensor_resizeAs", self._h, other._h)
        return self

    # ---- host <-> device ---------------------------------------------------
    def copy(self, src) -> "ClTensor":
        if isinstance(src, ClTensor):
            _call("THClTensor_copy", self._h, src._h)
        else:
            self._upload(np.asarray(src, dtype=np.float32))
        return self

    def float(self) -> np.ndarray:
        """``clTensor:float()``: a host copy shaped like the tensor."""
        nd = self.nDimension()
        if nd <= 0:
            # no dimensions: an empty tensor, or a point tensor, whose one value ``s()`` reads; as in Lua,
            # the host copy of either has no elements
            return np.empty((0,), dtype=np.float32)
        shape = self.size()
        out = np.empty(shape if nd > 0 else (0,), dtype=np.float32)
        if out.size:
            sz = (C.c_long * max(out.ndim, 1))(*out.shape)
            ft = self._lib.THFloatTensor_newWithData(out.ctypes.data_as(C.c_void_p), out.size, 0, out.ndim, sz, None)
            try:
                _call("THFloatTensor_copyCl", ft, self._h)
            finally:
                self._lib.THFloatTensor_free(ft)
        return out

    _HOST_TYPES = {"Byte": (np.uint8, C.c_ubyte), "Char": (np.int8, C.c_byte), "Short": (np.int16, C.c_short),
                   "Int": (np.int32, C.c_int), "Double": (np.float64, C.c_double)}

    def _to_host_typed(self, name: str) -> np.ndarray:
        """``clTensor:double()`` / ``:int()`` / ``:byte()`` ...: through TH<Name>Tensor_copyCl."""
        dtype, _ = self._HOST_TYPES[name]
        shape = self.size() if self.nDimension() > 0 else (0,)
        out = np.empty(shape, dtype=dtype)
        if out.size:
            sz = (C.c_long * out.ndim)(*out.shape)
            ht = getattr(self._lib, f"TH{name}Tensor_newWithData")(out.ctypes.data_as(C.c_void_p), out.size, 0, out.ndim, sz, None)
            try:
                _call(f"TH{name}Tensor_copyCl", ht, self._h)
            finally:
                getattr(self._lib, f"TH{name}Tensor_free")(ht)
        return out

    def _from_host_typed(self, name: str, arr: np.ndarray) -> "ClTensor":
        dtype, _ = self._HOST_TYPES[name]
        arr = np.asarray(arr, dtype=dtype)
        strides = tuple(s // arr.itemsize for s in arr.strides)
        if any(s < 0 for s in strides) or not arr.flags.aligned:
            arr = np.ascontiguousarray(arr)
            strides = tuple(s // arr.itemsize for s in arr.strides)
        sz, st = (C.c_long * max(arr.ndim, 1))(*arr.shape), (C.c_long * max(arr.ndim, 1))(*strides)
        span = 1 + sum((n - 1) * s for n, s in zip(arr.shape, strides)) if arr.size else 0
        ht = getattr(self._lib, f"TH{name}Tensor_newWithData")(arr.ctypes.data_as(C.c_void_p), span, 0, arr.ndim, sz, st)
        try:
            _call(f"THClTensor_copy{name}", self._h, ht)
        finally:
            getattr(self._lib, f"TH{name}Tensor_free")(ht)
        return self

    def double(self) -> np.ndarray:
        return self._to_host_typed("Double")

    def int(self) -> np.ndarray:
        return self._to_host_typed("Int")

    def short(self) -> np.ndarray:
        return self._to_host_typed("Short")

    def char(self) -> np.ndarray:
        return self._to_host_typed("Char")

    def byte(self) -> np.ndarray:
        return self._to_host_typed("Byte")

    def copyFrom(self, arr: np.ndarray) -> "ClTensor":
        """``cl:copy(hostTensor)`` for a host array of any of TH's element types (element counts must match)."""
        kinds = {np.dtype(np.uint8): "Byte", np.dtype(np.int8): "Char", np.dtype(np.int16): "Short",
                 np.dtype(np.int32): "Int", np.dtype(np.float64): "Double"}
        arr = np.asarray(arr)
        if arr.dtype in kinds:
            return self._from_host_typed(kinds[arr.dtype], arr)
        return self.copy(arr)

    def long(self) -> np.ndarray:
        return self.float().astype(np.int64)

    def s(self) -> float:
        """Point tensor -> host scalar (``src/TensorMath.lua:938-941``)."""
        return float(_call("THClTensor_as_float", self._h))

    # ---- fills --------------------------------------------------------------
    def fill(self, value) -> "ClTensor":
        if isinstance(value, ClTensor):
            _call("THClTensor_fill_gpu", self._h, value._h)
        else:
            _call("THClTensor_fill", self._h, C.c_float(value))
        return self

    def zero(self) -> "ClTensor":
        _call("THClTensor_zero", self._h)
        return self

    # ---- pointwise: overloads as declared in src/TensorMath.lua ---------------
    def add(self, *args) -> "ClTensor":
        """``x:add(v)``, ``x:add(y)``, ``x:add(v, y)``, ``x:add(a, v)``, ``x:add(a, v, b)``, ``x:add(a, b)``."""
        src, rest = self, args
        if len(args) >= 2 and isinstance(args[0], ClTensor):
            src, rest = args[0], args[1:]
        if len(rest) == 1 and not isinstance(rest[0], ClTensor):
            _call("THClTensor_add", self._h, src._h, C.c_float(rest[0]))
        elif len(rest) == 1:
            _call("THClTensor_cadd", self._h, src._h, C.c_float(1.0), rest[0]._h)
        elif len(rest) == 2:
            _call("THClTensor_cadd", self._h, src._h, C.c_float(rest[0]), rest[1]._h)
        else:
            raise ClError("invalid arguments to add")
        return self

    def csub(self, *args) -> "ClTensor":
        src, rest = self, args
        if len(args) >= 2 and isinstance(args[0], ClTensor):
            src, rest = args[0], args[1:]
        if len(rest) == 1 and not isinstance(rest[0], ClTensor):
            _call("THClTensor_sub", self._h, src._h, C.c_float(rest[0]))
        elif len(rest) == 1:
            _call("THClTensor_csub", self._h, src._h, C.c_float(1.0), rest[0]._h)
        elif len(rest) == 2:
            _call("THClTensor_csub", self._h, src._h, C.c_float(rest[0]), rest[1]._h)
        else:
            raise ClError("invalid arguments to csub")
        return self

    def _scalar_or_point(self, cfn: str, args) -> "ClTensor":
        src, v = (self, args[0]) if len(args) == 1 else (args[0], args[1])
        if isinstance(v, ClTensor):
            _call(f"THClTensor_{cfn}_gpu", self._h, src._h, v._h)
        else:
            _call(f"THClTensor_{cfn}", self._h, src._h, C.c_float(v))
        return self

    def mul(self, *args) -> "ClTensor":
        return self._scalar_or_point("mul", args)

    def div(self, *args) -> "ClTensor":
        """``a:div(v)`` or ``a:div(pointTensor)`` (``src/TensorMath.lua:727-736``)."""
        return self._scalar_or_point("div", args)

    def _binary(self, cfn: str, args) -> "ClTensor":
        a, b = (self, args[0]) if len(args) == 1 else (args[0], args[1])
        _call(f"THClTensor_{cfn}", self._h, a._h, b._h)
        return self

    def cmul(self, *args) -> "ClTensor":
        return self._binary("cmul", args)

    def cdiv(self, *args) -> "ClTensor":
        return self._binary("cdiv", args)

    def addcmul(self, *args) -> "ClTensor":
        t, rest = (self, args) if not isinstance(args[0], ClTensor) or len(args) == 2 else (args[0], args[1:])
        v, a, b = (1.0, rest[0], rest[1]) if len(rest) == 2 else rest
        _call("THClTensor_addcmul", self._h, t._h, C.c_float(v), a._h, b._h)
        return self

    def addcdiv(self, *args) -> "ClTensor":
        t, rest = (self, args) if not isinstance(args[0], ClTensor) or len(args) == 2 else (args[0], args[1:])
        v, a, b = (1.0, rest[0], rest[1]) if len(rest) == 2 else rest
        _call("THClTensor_addcdiv", self._h, t._h, C.c_float(v), a._h, b._h)
        return self

    def _unary(self, cfn: str, src: Optional["ClTensor"]) -> "ClTensor":
        _call(f"THClTensor_{cfn}", self._h, (src or self)._h)
        return self

    def sqrt(self, src=None): return self._unary("sqrt", src)
    def abs(self, src=None): return self._unary("abs", src)
    def neg(self, src=None): return self._unary("neg", src)
    def cinv(self, src=None): return self._unary("cinv", src)
    def exp(self, src=None): return self._unary("exp", src)
    def log(self, src=None): return self._unary("log", src)
    def tanh(self, src=None): return self._unary("tanh", src)
    def sigmoid(self, src=None): return self._unary("sigmoid", src)
    def floor(self, src=None): return self._unary("floor", src)
    def ceil(self, src=None): return self._unary("ceil", src)

    def log1p(self, src=None): return self._unary("log1p", src)
    def cos(self, src=None): return self._unary("cos", src)
    def acos(self, src=None): return self._unary("acos", src)
    def cosh(self, src=None): return self._unary("cosh", src)
    def sin(self, src=None): return self._unary("sin", src)
    def asin(self, src=None): return self._unary("asin", src)
    def sinh(self, src=None): return self._unary("sinh", src)
    def tan(self, src=None): return self._unary("tan", src)
    def atan(self, src=None): return self._unary("atan", src)
    def round(self, src=None): return self._unary("round", src)
    def sign(self, src=None): return self._unary("sign", src)

    def pow(self, *args) -> "ClTensor":
        """``x:pow(v)`` in place, ``res:pow(src, v)``, and ``res:pow(v, src)`` = v ^ src
        (``src/TensorMath.lua:1025-1033``)."""
        if len(args) == 1:
            _call("THClTensor_pow", self._h, self._h, C.c_float(args[0]))
        elif isinstance(args[0], ClTensor):
            _call("THClTensor_pow", self._h, args[0]._h, C.c_float(args[1]))
        else:
            _call("THClTensor_tpow", self._h, C.c_float(args[0]), args[1]._h)
        return self

    def cpow(self, *args) -> "ClTensor":
        return self._binary("cpow", args)

    def clamp(self, *args) -> "ClTensor":
        """``x:clamp(lo, hi)`` in place or ``res:clamp(src, lo, hi)``."""
        src, lo, hi = (self,) + tuple(args) if len(args) == 2 else args
        _call("THClTensor_clamp", self._h, src._h, C.c_float(lo), C.c_float(hi))
        return self

    def atan2(self, *args) -> "ClTensor":
        """``x:atan2(y)`` = atan2(x, y) in place, or ``res:atan2(a, b)``."""
        a, b = (self, args[0]) if len(args) == 1 else args
        _call("THClTensor_atan2", self._h, a._h, b._h)
        return self

    def _cminmax(self, name: str, args) -> "ClTensor":
        src, other = (self, args[0]) if len(args) == 1 else args
        if isinstance(other, ClTensor):
            _call(f"THClTensor_{name}", self._h, src._h, other._h)
        else:
            _call(f"THClTensor_{name}Value", self._h, src._h, C.c_float(other))
        return self

    def cmax(self, *args) -> "ClTensor":
        return self._cminmax("cmax", args)

    def cmin(self, *args) -> "ClTensor":
        return self._cminmax("cmin", args)

    def _compare(self, name: str, args) -> "ClTensor":
        """``a:lt(v)`` / ``a:lt(b)`` give a new 0/1 tensor; ``res:lt(a, v)`` / ``res:lt(a, b)``
        write into res (``src/TensorMath.lua:1052-1062``).  A 0-dim ClTensor on the right
        is a point tensor: the comparison reads it on the device."""
        res, src, other = (ClTensor(), self, args[0]) if len(args) == 1 else (self, args[0], args[1])
        if isinstance(other, ClTensor) and other.nDimension() == 0:
            _call(f"THClTensor_{name}PointTensor", res._h, src._h, other._h)
        elif isinstance(other, ClTensor):
            _call(f"THClTensor_{name}Tensor", res._h, src._h, other._h)
        else:
            _call(f"THClTensor_{name}Value", res._h, src._h, C.c_float(other))
        return res

    def lt(self, *args): return self._compare("lt", args)
    def gt(self, *args): return self._compare("gt", args)
    def le(self, *args): return self._compare("le", args)
    def ge(self, *args): return self._compare("ge", args)
    def eq(self, *args): return self._compare("eq", args)
    def ne(self, *args): return self._compare("ne", args)

    def maskedFill(self, mask, value: float) -> "ClTensor":
        if isinstance(mask, ClTensor):
            _call("THClTensor_maskedFill", self._h, mask._h, C.c_float(value))
        else:
            self._with_byte_mask(mask, lambda m: _call("THClTensor_maskedFillByte", self._h, m, C.c_float(value)))
        return self

    # ---- user expressions ---------------------------------------------------
    def apply_on_gpu(self, expr: str) -> "ClTensor":
        _call("THClTensor_apply", self._h, expr.encode())
        return self

    def map_on_gpu(self, other: "ClTensor", expr: str) -> "ClTensor":
        _call("THClTensor_map", self._h, other._h, expr.encode())
        return self

    def map2_on_gpu(self, a: "ClTensor", b: "ClTensor", expr: str) -> "ClTensor":
        _call("THClTensor_map2", self._h, a._h, b._h, expr.encode())
        return self

    apply2_on_gpu = map_on_gpu
    apply3_on_gpu = map2_on_gpu

    # ---- reductions -----------------------------------------------------------
    def _reduce(self, name: str, args):
        """``a:sum()`` -> number; ``res:sum(a)`` -> point tensor in res; ``a:sum(dim)`` -> new tensor."""
        if len(args) == 0:
            return float(_call(f"THClTensor_{name}all", self._h))
        if len(args) == 1 and isinstance(args[0], ClTensor):
            _call(f"THClTensor_{name}all_gpu", self._h, args[0]._h)
            return self
        raise ClError(f"invalid arguments to {name}")

    def _along(self, name: str, args):
        """``a:sum(dim)`` -> new tensor; ``res:sum(a, dim)`` -> res (the result slot first, as the wrapper
        table orders them: ``src/TensorMath.lua:943-953``); anything else is a whole-tensor form."""
        if len(args) == 1 and not isinstance(args[0], ClTensor):
            res = ClTensor()
            _call(f"THClTensor_{name}", res._h, self._h, C.c_long(args[0] - 1))
            return res
        if len(args) == 2 and isinstance(args[0], ClTensor) and not isinstance(args[1], ClTensor):
            _call(f"THClTensor_{name}", self._h, args[0]._h, C.c_long(args[1] - 1))
            return self
        return self._reduce(name, args)

    def sum(self, *args):
        return self._along("sum", args)

    def prod(self, *args):
        return self._along("prod", args)

    def _scan(self, name: str, args):
        """``a:cumsum()`` / ``a:cumsum(dim)`` -> new tensor (dim defaults to 1); ``res:cumsum(a, dim)``
        (``src/TensorMath.lua:955-961``)."""
        if len(args) >= 1 and isinstance(args[0], ClTensor):
            res, src, dim = self, args[0], (args[1] if len(args) > 1 else 1)
        else:
            res, src, dim = ClTensor(), self, (args[0] if args else 1)
        _call(f"THClTensor_{name}", res._h, src._h, C.c_long(dim - 1))
        return res

    def cumsum(self, *args):
        return self._scan("cumsum", args)

    def cumprod(self, *args):
        return self._scan("cumprod", args)

    def mean(self, *args):
        """``a:mean()`` -> number, ``a:mean(dim)`` -> new tensor (``src/TensorMath.lua:1104-1111``)."""
        if len(args) == 0:
            return float(_call("THClTensor_meanall", self._h))
        if len(args) == 2:                                    # res:mean(a, dim)
            _call("THClTensor_mean", self._h, args[0]._h, C.c_long(args[1] - 1))
            return self
        res = ClTensor()
        _call("THClTensor_mean", res._h, self._h, C.c_long(args[0] - 1))
        return res

    def norm(self, *args):
        """``a:norm()``, ``a:norm(p)`` -> number; ``a:norm(p, dim)`` -> new tensor."""
        if len(args) <= 1:
            return float(_call("THClTensor_normall", self._h, C.c_float(args[0] if args else 2.0)))
        res = ClTensor()
        _call("THClTensor_norm", res._h, self._h, C.c_float(args[0]), C.c_long(args[1] - 1))
        return res

    def _logical(self, name: str, args):
        if len(args) == 0:
            return bool(_call(f"THClTensor_logical{name}", self._h))
        _call(f"THClTensor_logical{name}_gpu", self._h, args[0]._h)
        return self

    def all(self, *args):
        """``a:all()`` -> boolean; ``res:all(a)`` leaves 1 / 0 in the point tensor res."""
        return self._logical("all", args)

    def any(self, *args):
        return self._logical("any", args)

    def _minmax(self, name: str, args):
        if len(args) == 1 and not isinstance(args[0], ClTensor):
            values, indices = ClTensor(), ClTensor()
            _call(f"THClTensor_{name}", values._h, indices._h, self._h, C.c_long(args[0] - 1))
            return values, indices
        if len(args) == 3 and isinstance(args[0], ClTensor) and isinstance(args[1], ClTensor):
            # values:max(indices, src, dim): both results into tensors that exist (src/TensorMath.lua:975-988)
            _call(f"THClTensor_{name}", self._h, args[0]._h, args[1]._h, C.c_long(args[2] - 1))
            return self, args[0]
        return self._reduce(name, args)

    def max(self, *args):
        """``a:max()`` -> number; ``a:max(dim)`` -> (values, 1-based indices as ClTensor)."""
        return self._minmax("max", args)

    def min(self, *args):
        return self._minmax("min", args)

    def max_long(self, dim: int) -> Tuple["ClTensor", np.ndarray]:
        """values plus int64 1-based indices (what ``indices:long()`` gives in Lua)."""
        return self._minmax_long("maxLong", dim)

    def min_long(self, dim: int) -> Tuple["ClTensor", np.ndarray]:
        return self._minmax_long("minLong", dim)

    def _minmax_long(self, cfn: str, dim: int):
        shape = [1 if d == dim - 1 else s for d, s in enumerate(self.size())]
        idx = np.zeros(shape, dtype=np.int64)
        sz = _long_storage(shape)
        lt = self._lib.THLongTensor_newWithSize(sz, None)
        self._lib.THLongStorage_free(sz)
        values = ClTensor()
        try:
            _call(f"THClTensor_{cfn}", values._h, lt, self._h, C.c_long(dim - 1))
            t = C.cast(lt, C.POINTER(_LongTensorStruct)).contents
            n = int(np.prod(shape))
            idx.reshape(-1)[:] = np.ctypeslib.as_array(t.storage.contents.data, shape=(n,))
        finally:
            self._lib.THLongTensor_free(lt)
        return values, idx

    # ---- blas -------------------------------------------------------------------
    def addmm(self, *args) -> "ClTensor":
        """``r:addmm([beta,] [t,] [alpha,] m1, m2)`` (``src/TensorMath.lua:896-929``)."""
        nums = [a for a in args if not isinstance(a, ClTensor)]
        tens = [a for a in args if isinstance(a, ClTensor)]
        if len(tens) == 2:
            t, m1, m2 = self, tens[0], tens[1]
        elif len(tens) == 3:
            t, m1, m2 = tens
        else:
            raise ClError("invalid arguments to addmm")
        if len(nums) == 0:
            beta, alpha = 1.0, 1.0
        elif len(nums) == 1:
            beta, alpha = 1.0, nums[0]
        else:
            beta, alpha = nums[0], nums[1]
        _call("THClTensor_addmm", self._h, C.c_float(beta), t._h, C.c_float(alpha), m1._h, m2._h)
        return self

    # ---- indexed movement (dims and indices 1-based, as in Lua) ---------------------
    def _with_index(self, cfn: str, index, call):
        """Runs ``call(name, handle)`` with a device index tensor, or a host LongTensor
        built from a list / integer array (the ``_long`` entry points)."""
        if isinstance(index, ClTensor):
            return call(f"THClTensor_{cfn}", index._h)
        lt = _long_vector(index)
        try:
            return call(f"THClTensor_{cfn}_long", lt)
        finally:
            self._lib.THLongTensor_free(lt)

    def index(self, *args) -> "ClTensor":
        """``a:index(dim, idx)`` -> new tensor; ``res:index(a, dim, idx)``."""
        res, src, dim, idx = (ClTensor(), self) + tuple(args) if len(args) == 2 else (self,) + tuple(args)
        self._with_index("indexSelect", idx, lambda fn, h: _call(fn, res._h, src._h, C.c_int(dim - 1), h))
        return res

    def indexCopy(self, dim: int, idx, src: "ClTensor") -> "ClTensor":
        self._with_index("indexCopy", idx, lambda fn, h: _call(fn, self._h, C.c_int(dim - 1), h, src._h))
        return self

    def indexFill(self, dim: int, idx, value: float) -> "ClTensor":
        self._with_index("indexFill", idx, lambda fn, h: _call(fn, self._h, C.c_int(dim - 1), h, C.c_float(value)))
        return self

    def gather(self, *args) -> "ClTensor":
        """``a:gather(dim, index)`` -> new tensor; ``res:gather(a, dim, index)``."""
        res, src, dim, idx = (ClTensor(), self) + tuple(args) if len(args) == 2 else (self,) + tuple(args)
        _call("THClTensor_gather", res._h, src._h, C.c_long(dim - 1), idx._h)
        return res

    def scatter(self, dim: int, index: "ClTensor", src) -> "ClTensor":
        """``a:scatter(dim, index, src)`` with a tensor or a number."""
        if isinstance(src, ClTensor):
            _call("THClTensor_scatter", self._h, C.c_long(dim - 1), index._h, src._h)
        else:
            _call("THClTensor_scatterFill", self._h, C.c_long(dim - 1), index._h, C.c_float(src))
        return self

    def maskedSelect(self, *args) -> "ClTensor":
        """``a:maskedSelect(mask)`` -> new vector; ``res:maskedSelect(a, mask)``."""
        res, src, mask = (ClTensor(), self, args[0]) if len(args) == 1 else (self, args[0], args[1])
        if isinstance(mask, ClTensor):
            _call("THClTensor_maskedSelect", res._h, src._h, mask._h)
        else:
            self._with_byte_mask(mask, lambda m: _call("THClTensor_maskedSelectByte", res._h, src._h, m))
        return res

    def maskedCopy(self, mask, src: "ClTensor") -> "ClTensor":
        if isinstance(mask, ClTensor):
            _call("THClTensor_maskedCopy", self._h, mask._h, src._h)
        else:
            self._with_byte_mask(mask, lambda m: _call("THClTensor_maskedCopyByte", self._h, m, src._h))
        return self

    def _with_byte_mask(self, mask, call):
        """A host ``torch.ByteTensor`` mask (numpy uint8 / bool array): the ``*Byte`` entry points."""
        arr = np.ascontiguousarray(np.asarray(mask).astype(np.uint8))
        sz = (C.c_long * max(arr.ndim, 1))(*arr.shape)
        bt = self._lib.THByteTensor_newWithData(arr.ctypes.data_as(C.c_void_p), arr.size, 0, arr.ndim, sz, None)
        try:
            return call(bt)
        finally:
            self._lib.THByteTensor_free(bt)

    def dot(self, other: "ClTensor") -> float:
        """``a:dot(b)`` (``src/TensorMath.lua:932-936``)."""
        return float(_call("THClTensor_dot", self._h, other._h))

    def _addblas(self, cfn: str, args) -> "ClTensor":
        """``r:addmv([beta,] [t,] [alpha,] mat, vec)`` and ``r:addr([beta,] [t,] [alpha,] v1, v2)``
        (``src/TensorMath.lua:896-929``)."""
        nums = [a for a in args if not isinstance(a, ClTensor)]
        tens = [a for a in args if isinstance(a, ClTensor)]
        if len(tens) == 2:
            t, a, b = self, tens[0], tens[1]
        elif len(tens) == 3:
            t, a, b = tens
        else:
            raise ClError(f"invalid arguments to {cfn}")
        beta, alpha = (1.0, 1.0) if not nums else ((1.0, nums[0]) if len(nums) == 1 else (nums[0], nums[1]))
        _call(f"THClTensor_{cfn}", self._h, C.c_float(beta), t._h, C.c_float(alpha), a._h, b._h)
        return self

    def addmv(self, *args) -> "ClTensor":
        return self._addblas("addmv", args)

    def addr(self, *args) -> "ClTensor":
        return self._addblas("addr", args)

    # ---- random fills (src/Random.lua:6-24): drawn on the host, then copied over ----------
    def uniform(self, a: float = 0.0, b: float = 1.0) -> "ClTensor":
        vals = _uniform01(self.nElement()) * (b - a) + a
        return self.copy(ClTensor(vals.astype(np.float32).reshape(self.size())))

    def bernoulli(self, p: float = 0.5) -> "ClTensor":
        vals = (_uniform01(self.nElement()) <= p).astype(np.float32)
        return self.copy(ClTensor(vals.reshape(self.size())))

    def normal(self, mean: float = 0.0, stdv: float = 1.0) -> "ClTensor":
        n = self.nElement()
        u1, u2 = _uniform01(n), _uniform01(n)
        vals = np.sqrt(-2.0 * np.log(1.0 - u2)) * np.cos(2.0 * np.pi * u1) * stdv + mean
        return self.copy(ClTensor(vals.astype(np.float32).reshape(self.size())))

    # ---- Lua operators (src/TensorOperator.c:5-250): each makes a new tensor ------------
    def _copy_of(self) -> "ClTensor":
        r = ClTensor(device=_call("THClTensor_getDevice", self._h))
        _call("THClTensor_resizeAs", r._h, self._h)
        _call("THClTensor_copy", r._h, self._h)
        return r

    def __add__(self, other) -> "ClTensor":
        r = self._copy_of()
        if isinstance(other, ClTensor):
            _call("THClTensor_cadd", r._h, r._h, C.c_float(1.0), other._h)
        else:
            _call("THClTensor_add", r._h, r._h, C.c_float(other))
        return r

    __radd__ = __add__

    def __sub__(self, other) -> "ClTensor":
        r = self._copy_of()
        if isinstance(other, ClTensor):
            _call("THClTensor_cadd", r._h, r._h, C.c_float(-1.0), other._h)
        else:
            _call("THClTensor_add", r._h, r._h, C.c_float(-other))
        return r

    def __rsub__(self, number) -> "ClTensor":
        """``number - tensor``: a tensor filled with the number, then ``cadd`` with -1."""
        r = ClTensor(device=_call("THClTensor_getDevice", self._h))
        _call("THClTensor_resizeAs", r._h, self._h)
        _call("THClTensor_fill", r._h, C.c_float(number))
        _call("THClTensor_cadd", r._h, r._h, C.c_float(-1.0), self._h)
        return r

    def __neg__(self) -> "ClTensor":
        r = self._copy_of()
        _call("THClTensor_mul", r._h, r._h, C.c_float(-1.0))
        return r

    def __mul__(self, other):
        """number: scaled copy; vector * vector: dot (a number); matrix * vector: mv; matrix * matrix: mm."""
        if not isinstance(other, ClTensor):
            r = self._copy_of()
            _call("THClTensor_mul", r._h, r._h, C.c_float(other))
            return r
        dt, ds = self.nDimension(), other.nDimension()
        if dt == 1 and ds == 1:
            return self.dot(other)
        if dt == 2 and ds == 1:
            return mv(self, other)
        if dt == 2 and ds == 2:
            r = ClTensor(self.size(1), other.size(2)).zero()
            _call("THClTensor_addmm", r._h, C.c_float(1.0), r._h, C.c_float(1.0), self._h, other._h)
            return r
        raise ClError(f"multiplication between {dt}D and {ds}D tensors not yet supported")

    def __rmul__(self, number) -> "ClTensor":
        return self.__mul__(number)

    def __truediv__(self, number) -> "ClTensor":
        """``tensor / number``: a copy multiplied by ``1 / number`` (the reciprocal is taken in double)."""
        if isinstance(number, ClTensor):
            raise ClError("number expected")
        r = self._copy_of()
        _call("THClTensor_mul", r._h, r._h, C.c_float(1.0 / number))
        return r

    def __str__(self):
        """``tostring(clTensor)``: the host copy in Torch7's text form."""
        from .printing import tensor_tostring
        return tensor_tostring(self.float() if self.nDimension() > 0 else np.zeros(()), "torch.ClTensor")

    def __repr__(self):
        return f"ClTensor(size={self.size()}, stride={self.stride()})"


def mm(a: ClTensor, b: ClTensor) -> ClTensor:
    """``torch.mm(a, b)``: zeroed result, then addmm with beta 0 (``src/TensorMath.lua:867-893``)."""
    r = ClTensor(a.size(1), b.size(2)).zero()
    _call("THClTensor_addmm", r._h, C.c_float(0.0), r._h, C.c_float(1.0), a._h, b._h)
    return r


def mv(mat: ClTensor, vec: ClTensor) -> ClTensor:
    """``torch.mv(mat, vec)``: zeroed result, then addmv (``src/TensorMath.lua:800-825``)."""
    r = ClTensor(mat.size(1)).zero()
    _call("THClTensor_addmv", r._h, C.c_float(1.0), r._h, C.c_float(1.0), mat._h, vec._h)
    return r


def ger(v1: ClTensor, v2: ClTensor) -> ClTensor:
    """``torch.ger(v1, v2)``: zeroed result, then addr (``src/TensorMath.lua:869-894``)."""
    r = ClTensor(v1.size(1), v2.size(1)).zero()
    _call("THClTensor_addr", r._h, C.c_float(1.0), r._h, C.c_float(1.0), v1._h, v2._h)
    return r


class _HostStorageStruct(C.Structure):  # TH<Type>Storage: data*, size, refcount, flag, allocator, allocatorContext, view
    _fields_ = [("data", C.c_void_p), ("size", C.c_long), ("refcount", C.c_int), ("flag", C.c_char),
                ("allocator", C.c_void_p), ("allocatorContext", C.c_void_p), ("view", C.c_void_p)]


class ClStorage:
    """``torch.ClStorage``: ``ClStorage()``, ``ClStorage(n)``, ``ClStorage{...}`` (a list), with ``fill``,
    ``resize``, ``copy`` (from another ClStorage or a host array: ``torch.Storage`` in the Lua tests),
    ``s[i]`` / ``s[i] = v`` (1-based), ``#s`` and ``tostring`` (src/torch/generic/Storage.cpp,
    src/test/unit_storage.lua:24-73)."""

    _COPY_IN = {np.dtype(np.float32): "Float", np.dtype(np.float64): "Double", np.dtype(np.int64): "Long",
                np.dtype(np.int32): "Int", np.dtype(np.int16): "Short", np.dtype(np.int8): "Char",
                np.dtype(np.uint8): "Byte"}

    def __init__(self, arg=None, device: int = 0):
        self._lib = state().lib
        if arg is None:
            self._h = _call("THClStorage_newv2", device)
        elif isinstance(arg, (int, np.integer)):
            self._h = _call("THClStorage_newWithSize", device, C.c_long(int(arg)))
        else:
            data = np.ascontiguousarray(arg, dtype=np.float32).reshape(-1)
            self._h = _call("THClStorage_newWithSize", device, C.c_long(data.size))
            self.copy(data)

    def __del__(self):
        try:
            if getattr(self, "_h", None) and _state is not None:
                self._lib.THClStorage_free(_state.ptr, self._h)
                self._h = None
        except Exception:
            pass

    def size(self) -> int:
        return int(_call("THClStorage_size", self._h))

    __len__ = size

    def fill(self, value: float) -> "ClStorage":
        _call("THClStorage_fill", self._h, C.c_float(value))
        return self

    def resize(self, n: int) -> "ClStorage":
        _call("THClStorage_resize", self._h, C.c_long(n))
        return self

    def copy(self, src) -> "ClStorage":
        """From a ClStorage, or from a host array of any of the seven element types (sizes must match)."""
        if isinstance(src, ClStorage):
            _call("THClStorage_copy", self._h, src._h)
            return self
        arr = np.ascontiguousarray(src)
        if arr.dtype not in self._COPY_IN:
            arr = arr.astype(np.float64)
        arr = arr.reshape(-1)
        host = _HostStorageStruct(arr.ctypes.data, arr.size, 1, b"\x00", None, None, None)
        _call("THClStorage_copy" + self._COPY_IN[arr.dtype], self._h, C.byref(host))
        return self

    def to_host(self, dtype=np.float32) -> np.ndarray:
        """``hostStorage:copy(clStorage)``: the elements as a host array of the given type."""
        out = np.zeros(self.size(), dtype=dtype)
        host = _HostStorageStruct(out.ctypes.data, out.size, 1, b"\x00", None, None, None)
        _call("TH" + self._COPY_IN[np.dtype(dtype)] + "Storage_copyCl", C.byref(host), self._h)
        return out

    def __getitem__(self, i: int) -> float:
        fn = self._lib.THClStorage_get
        fn.restype = C.c_float
        return float(_call("THClStorage_get", self._h, C.c_long(i - 1)))

    def __setitem__(self, i: int, value: float) -> None:
        _call("THClStorage_set", self._h, C.c_long(i - 1), C.c_float(value))

    def __str__(self) -> str:
        from .printing import storage_tostring
        return storage_tostring(self.to_host(), "torch.ClStorage")


class ClKernel:
    """``torch.ClKernel({input={...}, output={...}, inout={...}, src=..., funcs=..., name=...})``
    and ``k:run(params [, {numWorkgroups=, workgroupSize=}])`` (``src/UserKernel.cpp:217-383``).
    Argument types are ``'int'``, ``'float'`` and ``'ClTensor'`` / ``'torch.ClTensor'``."""

    _TYPES = {"int": 0, "float": 1, "ClTensor": 2, "torch.ClTensor": 2}

    def __init__(self, spec: dict):
        if not isinstance(spec, dict):
            raise ClError("First parameter to torch.ClKernel should be a table")
        unknown = set(spec) - {"input", "output", "inout", "src", "funcs", "name"}
        if unknown:
            raise ClError(f"Parameter {sorted(unknown)[0]} not recognized")
        self._args = []
        for direction, key in ((0, "input"), (1, "output"), (2, "inout")):
            for name, typename in (spec.get(key) or {}).items():
                if typename not in self._TYPES:
                    raise ClError(f"Unrecognized typename {typename}")
                self._args.append((name, self._TYPES[typename], direction))
        n = len(self._args)
        names = (C.c_char_p * max(n, 1))(*[a[0].encode() for a in self._args])
        types = (C.c_int * max(n, 1))(*[a[1] for a in self._args])
        dirs = (C.c_int * max(n, 1))(*[a[2] for a in self._args])
        name = spec.get("name")
        funcs = spec.get("funcs")
        self._lib = state().lib
        self._src = spec.get("src") or ""
        self._h = _call("THClKernel_new", name.encode() if name else None, self._src.encode(),
                        funcs.encode() if funcs else None, C.c_int(n), names, types, dirs)
        if not self._h:
            raise ClError("kernel construction failed")

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                self._lib.THClKernel_free(None, self._h)
                self._h = None
        except Exception:
            pass

    def getRenderedKernel(self) -> str:
        return self._lib.THClKernel_getRenderedKernel(self._h).decode()

    def getRawKernel(self) -> str:
        """The body as it was given (src/UserKernel.cpp:304-308)."""
        return self._src

    def print(self) -> str:
        """``k:print()`` (src/UserKernel.cpp:292-303): both sources under the reference's headings."""
        text = ("Original source\n===============\n" + self._src + "\n\n" +
                "Generated source\n================\n" + self.getRenderedKernel() + "\n")
        print(text, end="")
        return text

    def run(self, params: dict, options: Optional[dict] = None) -> None:
        options = options or {}
        unknown = set(options) - {"numWorkgroups", "workgroupSize"}
        if unknown:
            raise ClError(f"option {sorted(unknown)[0]} not recognized")
        n = len(self._args)
        ints, floats = (C.c_int * max(n, 1))(), (C.c_float * max(n, 1))()
        tensors = (C.c_void_p * max(n, 1))()
        for i, (name, typ, _) in enumerate(self._args):
            if name not in params:
                raise ClError(f"missing value for parameter {name}")
            v = params[name]
            if typ == 2:
                if not isinstance(v, ClTensor):
                    raise ClError(f"parameter {name} must be a ClTensor")
                tensors[i] = v._h
            elif typ == 0:
                ints[i] = int(v)
            else:
                floats[i] = float(v)
        _call("THClKernel_run", self._h, ints, floats, tensors, C.c_long(int(options.get("numWorkgroups", 0))),
              C.c_long(int(options.get("workgroupSize", 0))))

