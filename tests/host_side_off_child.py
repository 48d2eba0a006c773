"""Run by tests/test_gpu_configs.py in a process of its own with THCL_HOST_COPY_THREADS=0 and THCL_SCALAR_SPIN_US=0
(both are read when the first device context is opened): the piece-boundary copies and the scalar-returning calls
with the library's host threads and its polling switched off.  Prints `host side off ok` and the thread count."""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import cltorch_amd as cl  # noqa: E402
from cltorch_amd.tensor import _call  # noqa: E402

F = np.float32
assert os.environ.get("THCL_HOST_COPY_THREADS") == "0" and os.environ.get("THCL_SCALAR_SPIN_US") == "0"


def threads():
    return len(os.listdir("/proc/self/task"))


lib = cl.state().lib
before = threads()
for n in (511, 512, 513, 16385, (1 << 18) + 3, (2 << 18) + 1, (9 << 18) - 5, (33 << 18) + 12, 64 << 18, (70 << 18) + 7):
    rng = np.random.RandomState(n % 1000)
    a = rng.standard_normal(n).astype(F)
    t = cl.ClTensor(a)
    t.mul(2.0)
    assert np.array_equal(t.float().view(np.uint32), (a * F(2.0)).view(np.uint32)), n
    into = np.full(n, -7.0, dtype=F)
    sz = (C.c_long * 1)(n)
    ft = lib.THFloatTensor_newWithData(into.ctypes.data_as(C.c_void_p), n, 0, 1, sz, None)
    _call("THFloatTensor_copyCl", ft, t._h)
    assert np.array_equal(into, a * F(2.0)), n
    into[:] = (np.arange(n) % 977).astype(F)
    _call("THClTensor_copyFloat", t._h, ft)
    lib.THFloatTensor_free(ft)
    # scalars come back through a wait for the stream
    assert t.sum() == float(np.float32(float((np.arange(n) % 977).sum()))), n
    assert t.max() == float(min(n - 1, 976)) and t.min() == 0.0
    if n <= (9 << 18):
        d = rng.standard_normal(n) * 50.0          # converted on the calling thread
        for dt in (np.float64, np.int64, np.int16, np.uint8):
            h = (np.abs(d) if dt == np.uint8 else d).astype(dt)
            s = cl.ClStorage(n)
            s.copy(h)
            assert np.array_equal(s.to_host(), h.astype(F)), (n, dt)
            assert np.array_equal(s.to_host(dt), h.astype(F).astype(dt)), (n, dt)
x = cl.ClTensor(np.arange(1000, dtype=F))
assert x.dot(x) == float(np.float32(float((np.arange(1000, dtype=np.float64) ** 2).sum())))
started = threads() - before
print("host side off ok; threads started by the copies:", started)
assert started == 0, started
