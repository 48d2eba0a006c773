"""Helpers for the GPU parity tests: the same strided view on both sides."""
import numpy as np

import oracle
from oracle import View


def _inside(storage_size, offset, sizes, strides):
    last = offset + sum((s - 1) * t for s, t in zip(sizes, strides))
    assert 0 <= offset and last < storage_size, f"view reaches element {last} of a storage of {storage_size}"


class Pair:
    """A flat storage on host (oracle View) and on the device (ClTensor over the same layout)."""

    def __init__(self, cl, storage: np.ndarray, offset=0, sizes=None, strides=None):
        storage = np.ascontiguousarray(storage, dtype=np.float32).reshape(-1)
        self.cl = cl
        self.host_storage = storage.copy()
        self.flat = cl.ClTensor(storage)           # 1-d dense tensor owning the device storage
        if sizes is None:
            sizes, strides = (storage.size,), (1,)
        _inside(storage.size, offset, sizes, strides)
        self.view = View(self.host_storage, offset, sizes, strides)
        self.dev = self.flat.strided(sizes, strides, offset + 1)

    @staticmethod
    def dense(cl, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        v = View.contiguous(arr)
        return Pair(cl, v.storage, 0, v.sizes, v.strides)

    def derive(self, view: View) -> "Pair":
        """Another view of the same two storages."""
        p = object.__new__(Pair)
        p.cl, p.host_storage, p.flat = self.cl, self.host_storage, self.flat
        _inside(self.host_storage.size, view.offset, view.sizes, view.strides)
        p.view = View(self.host_storage, view.offset, view.sizes, view.strides)
        p.dev = self.flat.strided(view.sizes, view.strides, view.offset + 1)
        return p

    def transpose(self, a, b):
        return self.derive(self.view.transpose(a, b))

    def narrow(self, d, first, size):
        return self.derive(self.view.narrow(d, first, size))

    def step(self, d, k):
        return self.derive(self.view.step(d, k))

    def device_storage(self) -> np.ndarray:
        return self.flat.float()


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).reshape(-1).view(np.uint32)


def assert_bit_equal(got, want, what=""):
    """Bit-for-bit, except that any NaN matches any NaN (payload/sign of an
    invalid-operation NaN is not part of the arithmetic being compared)."""
    got = np.ascontiguousarray(got, dtype=np.float32).reshape(-1)
    want = np.ascontiguousarray(want, dtype=np.float32).reshape(-1)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    gn, wn = np.isnan(got), np.isnan(want)
    assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
    ok = ~wn
    bad = np.nonzero(got[ok].view(np.uint32) != want[ok].view(np.uint32))[0]
    assert bad.size == 0, f"{what}: {bad.size} of {got.size} elements differ, first at {bad[0]}: {got[ok][bad[0]]!r} vs {want[ok][bad[0]]!r}"
