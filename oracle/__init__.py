"""CPU oracle for the hot path: TEST INFRASTRUCTURE ONLY.

ctypes front-end of ``th_oracle.c`` (a restatement of the Torch7 ``TH``
FloatTensor semantics that the reference's own tests compare against, e.g.
``src/test/unit_tensor.lua:73-93``).  Only ``tests/``, ``__graft_entry__.smoke``
and the ``cpu_baseline`` leg of ``bench.py`` may import this package; the
shipped library never does.

What pins each function (see ``tests/test_oracle_*.py``):

* pointwise ops: closed form per element against numpy float32 arithmetic and
  the inputs of ``src/test/unit_tensor.lua:225-306``;
* collapse / contiguity / overlap rules: brute-force offset equality on random
  shapes and the worked layouts of the strided configurations;
* sum / prod: ``math.fsum`` (exactly rounded) and closed forms;
* max / min (+ indices): brute force, planted ties and NaNs;
* addmm: numpy float64 matmul and the integer matrices of
  ``src/test/unit_tensor.lua:413-438``;
* MT19937: the published first outputs for seed 5489 and numpy's
  ``RandomState`` raw stream.

Parity unpinned (no Torch7 here to confirm): the exact ``THRandom`` stream of
``torch.manualSeed`` (irrelevant: both sides consume the same arrays) and
TH's scalar ``div`` rounding (true division, restated from public TH sources).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libth_oracle.so")

OPS = dict(
    fill=0, copy=1, add_s=2, mul_s=3, div_s=4, cadd=5, cmul=6, cdiv=7, csub=8, sub_s=9,
    mulrecip_s=10, sqrt=11, neg=12, abs=13, cinv=14, addcmul=15, map2_c1=16, map_c2=17,
)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds)."""
    src = os.path.join(_HERE, "th_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.th_sumall.restype = C.c_double
        _lib.th_prodall.restype = C.c_double
        _lib.th_maxall.restype = C.c_float
        _lib.th_minall.restype = C.c_float
        _lib.th_num_threads.restype = C.c_int
    return _lib


@dataclass
class View:
    """A strided float32 view over a flat storage array (elements, not bytes)."""

    storage: np.ndarray
    offset: int
    sizes: Sequence[int]
    strides: Sequence[int]

    def __post_init__(self):
        assert self.storage.dtype == np.float32 and self.storage.ndim == 1
        self.sizes = tuple(int(s) for s in self.sizes)
        self.strides = tuple(int(s) for s in self.strides)

    @staticmethod
    def contiguous(arr: np.ndarray) -> "View":
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        st, z = [], 1
        for s in reversed(arr.shape):
            st.append(z)
            z *= s
        return View(arr.reshape(-1), 0, arr.shape, tuple(reversed(st)))

    @property
    def numel(self) -> int:
        if len(self.sizes) == 0:
            return 0
        return int(np.prod(self.sizes, dtype=np.int64))

    def cargs(self):
        nd = len(self.sizes)
        sz = (C.c_long * max(nd, 1))(*self.sizes)
        st = (C.c_long * max(nd, 1))(*self.strides)
        return (self.storage.ctypes.data_as(C.c_void_p), C.c_long(self.offset), C.c_int(nd), sz, st)

    def gather(self) -> np.ndarray:
        """Elements in logical order as a fresh array of shape ``sizes``."""
        v = np.lib.stride_tricks.as_strided(
            self.storage[self.offset:], shape=self.sizes, strides=tuple(4 * s for s in self.strides))
        return np.array(v, dtype=np.float32)

    def transpose(self, d0: int, d1: int) -> "View":
        sz, st = list(self.sizes), list(self.strides)
        sz[d0], sz[d1] = sz[d1], sz[d0]
        st[d0], st[d1] = st[d1], st[d0]
        return View(self.storage, self.offset, sz, st)

    def narrow(self, dim: int, first: int, size: int) -> "View":
        sz = list(self.sizes)
        sz[dim] = size
        return View(self.storage, self.offset + first * self.strides[dim], sz, self.strides)

    def step(self, dim: int, k: int) -> "View":
        """Every k-th element along ``dim`` (what ``unfold``/stride tricks give)."""
        sz, st = list(self.sizes), list(self.strides)
        sz[dim] = (sz[dim] + k - 1) // k
        st[dim] *= k
        return View(self.storage, self.offset, sz, st)


_NULLV = (C.c_void_p(None), C.c_long(0), C.c_int(0), (C.c_long * 1)(0), (C.c_long * 1)(0))


def pointwise(op: str, r: View, a: Optional[View] = None, b: Optional[View] = None, value: float = 0.0):
    """In place: r[i] = op(r[i], a[i], b[i], value)."""
    rc = lib().th_pointwise(C.c_int(OPS[op]), C.c_float(value), *r.cargs(),
                            *(a.cargs() if a is not None else _NULLV),
                            *(b.cargs() if b is not None else _NULLV))
    if rc != 0:
        raise ValueError("element count mismatch")


def sumall(v: View) -> float:
    """TH semantics: double accumulator; caller narrows to float."""
    return float(lib().th_sumall(*v.cargs()))


def prodall(v: View) -> float:
    return float(lib().th_prodall(*v.cargs()))


def maxall(v: View) -> float:
    return float(lib().th_maxall(*v.cargs()))


def minall(v: View) -> float:
    return float(lib().th_minall(*v.cargs()))


def reduce_dim(kind: str, v: View, dim: int):
    """Returns (values float32 of the reduced shape, 1-based int64 indices or None)."""
    k = dict(sum=0, prod=1, max=2, min=3)[kind]
    oshape = tuple(1 if d == dim else s for d, s in enumerate(v.sizes))
    out = np.empty(int(np.prod(oshape)), dtype=np.float32)
    idx = np.empty(out.size, dtype=np.int64) if k >= 2 else None
    rc = lib().th_reduce_dim(C.c_int(k), C.c_int(dim), *v.cargs(), out.ctypes.data_as(C.c_void_p),
                             idx.ctypes.data_as(C.c_void_p) if idx is not None else C.c_void_p(None))
    if rc != 0:
        raise ValueError("dimension out of range")
    return out.reshape(oshape), (idx.reshape(oshape) if idx is not None else None)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def addmm_f64(beta, t: View, alpha, m1: View, m2: View) -> np.ndarray:
    M, K = m1.sizes
    K2, N = m2.sizes
    assert K == K2 and tuple(t.sizes) == (M, N)
    r = np.empty((M, N), dtype=np.float64)
    lib().th_addmm_f64(_p(r), C.c_float(beta), C.c_void_p(t.storage.ctypes.data + 4 * t.offset),
                       C.c_long(t.strides[0]), C.c_long(t.strides[1]), C.c_float(alpha),
                       C.c_void_p(m1.storage.ctypes.data + 4 * m1.offset), C.c_long(m1.strides[0]), C.c_long(m1.strides[1]),
                       C.c_void_p(m2.storage.ctypes.data + 4 * m2.offset), C.c_long(m2.strides[0]), C.c_long(m2.strides[1]),
                       C.c_long(M), C.c_long(N), C.c_long(K))
    return r


def addmm_f64_sampled(rows, cols, beta, t: View, alpha, m1: View, m2: View) -> np.ndarray:
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    cols = np.ascontiguousarray(cols, dtype=np.int64)
    K = m1.sizes[1]
    r = np.empty(rows.size, dtype=np.float64)
    lib().th_addmm_f64_sampled(_p(r), C.c_long(rows.size), _p(rows), _p(cols), C.c_float(beta),
                               C.c_void_p(t.storage.ctypes.data + 4 * t.offset), C.c_long(t.strides[0]), C.c_long(t.strides[1]),
                               C.c_float(alpha),
                               C.c_void_p(m1.storage.ctypes.data + 4 * m1.offset), C.c_long(m1.strides[0]), C.c_long(m1.strides[1]),
                               C.c_void_p(m2.storage.ctypes.data + 4 * m2.offset), C.c_long(m2.strides[0]), C.c_long(m2.strides[1]),
                               C.c_long(K))
    return r


def collapse(sizes, strides, reduce_dim: int = -1):
    nd = len(sizes)
    sz = (C.c_long * max(nd, 1))(*sizes)
    st = (C.c_long * max(nd, 1))(*strides)
    csz = (C.c_long * 25)()
    cst = (C.c_long * 25)()
    k = lib().th_collapse(C.c_int(nd), sz, st, C.c_int(reduce_dim), csz, cst)
    return list(csz[:k]), list(cst[:k])


def is_contiguous(sizes, strides) -> bool:
    nd = len(sizes)
    return bool(lib().th_is_contiguous(C.c_int(nd), (C.c_long * max(nd, 1))(*sizes), (C.c_long * max(nd, 1))(*strides)))


def overlapping(sizes, strides) -> bool:
    nd = len(sizes)
    return bool(lib().th_overlapping(C.c_int(nd), (C.c_long * max(nd, 1))(*sizes), (C.c_long * max(nd, 1))(*strides)))


def mt_raw(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, dtype=np.uint32)
    lib().th_mt_raw(C.c_uint32(seed), C.c_long(n), _p(out))
    return out


def uniform(seed: int, n: int, lo: float = -1.0, hi: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().th_fill_uniform(C.c_uint32(seed), C.c_long(n), C.c_double(lo), C.c_double(hi), _p(out))
    return out


def normal(seed: int, n: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().th_fill_normal(C.c_uint32(seed), C.c_long(n), C.c_double(mean), C.c_double(std), _p(out))
    return out


def num_threads() -> int:
    return int(lib().th_num_threads())
