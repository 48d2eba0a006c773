"""The entry point that allocates nothing: THClTensor_sumall_gpu_noalloc against
THClTensor_sumall_gpu, through the C ABI.

Its arrival ticket and per-block partials sit in a static device array that keeps the
previous call's contents, so the calls come in pairs, the second on a smaller input:
left-over partials or a ticket that did not return to zero would show there.  The two
entry points run the same kernel on the same grid, so the results are compared bit for
bit, and against the CPU oracle within the 1e-5 relative bound of sums.  This file is
collected last so that a failure here hides no other test; it also passes alone in a
fresh process."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import View
from gpu_util import Pair

pytestmark = pytest.mark.gpu
F = np.float32


def _point(cl):
    """A point tensor that already owns its one-element storage."""
    p = cl.ClTensor()
    p.sum(cl.ClTensor(np.zeros(4, dtype=F)))
    assert p.nDimension() == 0
    return p


def _both(cl, src):
    from cltorch_amd.tensor import _call
    want, got = _point(cl), _point(cl)
    _call("THClTensor_sumall_gpu", want._h, src._h)
    before = cl.memoryStats()
    _call("THClTensor_sumall_gpu_noalloc", got._h, src._h)
    after = cl.memoryStats()
    assert after["device_mallocs"] == before["device_mallocs"] and after["cache_hits"] == before["cache_hits"]
    return F(want.s()), F(got.s())


def test_two_calls_in_a_row_the_second_smaller(cl):
    big = oracle.uniform(31, (1 << 24) + 3, 0.0, 1.0)
    small = oracle.uniform(32, 1000, -1.0, 1.0)
    for a in (big, small, big[: 1 << 20], small[:1]):
        A = cl.ClTensor(a)
        want, got = _both(cl, A)
        assert got.view(np.uint32) == want.view(np.uint32), (a.size, got, want)
        truth = oracle.sumall(View.contiguous(a))
        assert abs(float(got) - truth) <= 1e-5 * max(abs(truth), 1e-30), (a.size, got, truth)
    # closed forms: a left-over partial of the larger call would change these
    ones = cl.ClTensor(1 << 22).fill(1.0)
    assert _both(cl, ones)[1] == float(1 << 22)
    assert _both(cl, ones.narrow(1, 1, 7))[1] == 7.0


def test_strided_sources_and_repeats(cl):
    r, c = 1024, 768
    p = Pair.dense(cl, oracle.uniform(33, r * c).reshape(r, c))
    views = [p.transpose(0, 1), p.narrow(1, 5, 300), p.step(1, 3), p.narrow(0, 17, 2).narrow(1, 1, 5)]
    for v in views:
        want, got = _both(cl, v.dev)
        assert got.view(np.uint32) == want.view(np.uint32)
        truth = oracle.sumall(v.view)
        assert abs(float(got) - truth) <= 1e-5 * max(abs(truth), 1e-6)
    # the same call many times over: the ticket returns to zero every time
    ones = cl.ClTensor(1 << 20).fill(1.0)
    from cltorch_amd.tensor import _call
    outs = [_point(cl) for _ in range(50)]
    for o in outs:
        _call("THClTensor_sumall_gpu_noalloc", o._h, ones._h)
    assert all(o.s() == float(1 << 20) for o in outs)
    # the allocating entry point still works in between and afterwards
    assert ones.sum() == float(1 << 20)


def test_what_it_refuses(cl):
    from cltorch_amd.tensor import _call
    a = cl.ClTensor(np.ones(16, dtype=F))
    empty, vec = cl.ClTensor(), cl.ClTensor(3)
    with pytest.raises(cl.ClError, match="point tensor"):
        _call("THClTensor_sumall_gpu_noalloc", empty._h, a._h)                  # no storage yet: would have to allocate
    with pytest.raises(cl.ClError, match="point tensor"):
        _call("THClTensor_sumall_gpu_noalloc", vec._h, a._h)                    # would have to be resized
    # beyond the stated maximum: a stride-0 view names 2^31 elements without owning them
    huge = a.strided((1 << 16, 1 << 15), (0, 0))
    assert huge.nElement() == 1 << 31
    out = _point(cl)
    with pytest.raises(cl.ClError, match="at most"):
        _call("THClTensor_sumall_gpu_noalloc", out._h, huge._h)
    # maskedSelect / maskedCopy keep 32-bit offsets: 2^32 elements or more are refused before anything is allocated
    wide = a.strided((1 << 16, 1 << 16), (0, 0))
    with pytest.raises(cl.ClError, match="at most 2\\^32 - 1 elements"):
        cl.ClTensor().maskedSelect(wide, wide)
    # an empty source gives the identity element, and the library goes on working
    _call("THClTensor_sumall_gpu_noalloc", out._h, empty._h)
    assert out.s() == 0.0
    assert a.sum() == 16.0
