"""CPU restatement of the pointwise operator catalogue: TEST INFRASTRUCTURE.

Each entry follows the operator string the reference compiles
(src/lib/THClTensorMathPointwise.cpp:39-58,191-319, src/lib/THClTensorMath2.cpp:22-188,
src/lib/THClTensorMathCompare.cpp:26-82, src/lib/THClTensorMathCompareT.cpp:28-57,
src/lib/THClTensorMasked.cpp:29-38) evaluated in fp32 with numpy.  Exact
operators (compare, clamp, sign, round, cmax/cmin, maskedFill, integer powers
of small integers) are compared bit for bit; the transcendental ones within
the tolerance the reference's own tests use (src/test/unit_tensor.lua:73-93).
Pinned in tests/test_oracle.py by special values and identities.
"""
import numpy as np

F = np.float32


def _f(x):
    return np.asarray(x, dtype=F)


UNARY = {
    "log1p": np.log1p, "cos": np.cos, "acos": np.arccos, "cosh": np.cosh, "sin": np.sin, "asin": np.arcsin,
    "sinh": np.sinh, "tan": np.tan, "atan": np.arctan, "exp": np.exp, "log": np.log, "tanh": np.tanh,
    "floor": np.floor, "ceil": np.ceil, "sqrt": np.sqrt, "abs": np.abs,
}


def unary(name, x):
    x = _f(x)
    if name == "round":          # C round(): halves away from zero (numpy's rounds them to even)
        return np.trunc(x.astype(np.float64) + np.copysign(0.5, x.astype(np.float64))).astype(F)
    if name == "sign":           # (x > 0) - (x < 0)
        return ((x > 0).astype(np.int32) - (x < 0).astype(np.int32)).astype(F)
    with np.errstate(all="ignore"):
        return UNARY[name](x).astype(F)


def pown(x, n: int):
    """Repeated multiplication in fp32 (square and multiply), 1/x^|n| for negative n."""
    x = _f(x)
    r = np.ones_like(x)
    b = x.copy()
    e = abs(int(n))
    with np.errstate(all="ignore"):
        while e:
            if e & 1:
                r = (r * b).astype(F)
            b = (b * b).astype(F)
            e >>= 1
        return (F(1.0) / r).astype(F) if n < 0 else r


def pow_value(x, v: float):
    """src ^ v: integer-valued v goes through pown (src/lib/THClTensorMath2.cpp:28-35)."""
    if float(int(v)) == float(v):
        return pown(x, int(v))
    with np.errstate(all="ignore"):
        return np.power(_f(x), F(v)).astype(F)


def tpow(v: float, x):
    with np.errstate(all="ignore"):
        return np.power(F(v), _f(x)).astype(F)


def cpow(a, b):
    with np.errstate(all="ignore"):
        return np.power(_f(a), _f(b)).astype(F)


def clamp(x, lo, hi):
    """fmax(fmin(x, hi), lo): NaN-ignoring min then max."""
    return np.fmax(np.fmin(_f(x), F(hi)), F(lo))


def atan2(a, b):
    return np.arctan2(_f(a), _f(b)).astype(F)


def cmax(a, b):
    """OpenCL max(x, y): y if x < y else x."""
    a, b = _f(a), np.broadcast_to(_f(b), np.shape(a))
    return np.where(a < b, b, a).astype(F)


def cmin(a, b):
    """OpenCL min(x, y): y if y < x else x."""
    a, b = _f(a), np.broadcast_to(_f(b), np.shape(a))
    return np.where(b < a, b, a).astype(F)


_REL = {"lt": np.less, "gt": np.greater, "le": np.less_equal, "ge": np.greater_equal, "eq": np.equal, "ne": np.not_equal}


def compare(name, a, b):
    with np.errstate(invalid="ignore"):
        return _REL[name](_f(a), _f(b)).astype(F)


def masked_fill(x, mask, value):
    return np.where(_f(mask) != 0, F(value), _f(x)).astype(F)


# ------------------------------------------------------------- reductions / scans ---
def cumulate(x, axis: int, prod: bool = False):
    """Torch7's CPU cumsum / cumprod: a sequential fp64 running value, every
    output its rounding to fp32 (numpy's cumsum / cumprod on float64 run sequentially)."""
    x64 = np.asarray(x, dtype=np.float64)
    with np.errstate(all="ignore"):
        return (np.cumprod(x64, axis=axis) if prod else np.cumsum(x64, axis=axis)).astype(F)


def norm(x, p: float, axis=None):
    """p == 0 counts non-zero elements; otherwise (sum |x|^p)^(1/p) with fp64
    accumulation (TH's accreal), rounded to fp32 once per output."""
    x64 = np.abs(np.asarray(x, dtype=np.float64))
    keep = axis is not None
    if p == 0:
        return (x64 != 0).sum(axis=axis, keepdims=keep).astype(F)
    return np.power(np.power(x64, p).sum(axis=axis, keepdims=keep), 1.0 / p).astype(F)


def truth(x):
    """Element truth value of the reference's all / any reductions: (int)x != 0,
    i.e. truncation toward zero (src/lib/THClTensorMath.cpp:444-458)."""
    return np.trunc(_f(x)) != 0


# --------------------------------------------------------------- level 1 / 2 ---
def dot(a, b):
    """fp64 products and running sum, one rounding (the reference tests compare
    its clBLAS result with Torch7's CPU dot within 1e-4: src/test/unit_tensor.lua:413-461)."""
    return F(np.dot(np.asarray(a, dtype=np.float64).ravel(), np.asarray(b, dtype=np.float64).ravel()))


def addmv(beta, t, alpha, mat, vec):
    """beta * t + alpha * mat @ vec in fp64 (src/lib/THClTensorMathBlas.cpp:43-105)."""
    return beta * np.asarray(t, dtype=np.float64) + alpha * (np.asarray(mat, dtype=np.float64) @ np.asarray(vec, dtype=np.float64))


def addr(beta, t, alpha, v1, v2):
    """beta * t + alpha * outer(v1, v2) in fp64 (src/lib/THClTensorMathBlas.cpp:216-277)."""
    return beta * np.asarray(t, dtype=np.float64) + alpha * np.outer(np.asarray(v1, dtype=np.float64), np.asarray(v2, dtype=np.float64))


# ------------------------------------------------------------ indexed movement ---
# Torch7 CPU semantics (TH's sequential loops) behind the entry points of
# src/lib/THClTensorIndex.cpp, THClGather.cpp, THClScatter.cpp, THClTensorMasked.cpp.
# Indices are 1-based.
def index_select(src, dim, idx):
    return np.take(_f(src), np.asarray(idx, dtype=np.int64) - 1, axis=dim)


def index_copy(res, dim, idx, src):
    """res[.., idx[i], ..] = src[.., i, ..] in order of i: a repeated target keeps the last."""
    res = _f(res).copy()
    src = _f(src)
    for i, j in enumerate(np.asarray(idx, dtype=np.int64) - 1):
        sl = [slice(None)] * res.ndim
        sl[dim] = int(j)
        ss = [slice(None)] * res.ndim
        ss[dim] = i
        res[tuple(sl)] = src[tuple(ss)]
    return res


def index_fill(res, dim, idx, value):
    res = _f(res).copy()
    for j in np.asarray(idx, dtype=np.int64) - 1:
        sl = [slice(None)] * res.ndim
        sl[dim] = int(j)
        res[tuple(sl)] = F(value)
    return res


def gather(src, dim, index):
    return np.take_along_axis(_f(src), np.asarray(index, dtype=np.int64) - 1, axis=dim)


def scatter(res, dim, index, src):
    """res[index[i][j][k]][j][k] = src[i][j][k] (dim 0); src may be a number."""
    res = _f(res).copy()
    index = np.asarray(index, dtype=np.int64) - 1
    vals = np.broadcast_to(_f(src), index.shape)
    np.put_along_axis(res, index, vals, axis=dim)
    return res


def masked_select(src, mask):
    return _f(src).reshape(-1)[_f(mask).reshape(-1) != 0]


def masked_copy(res, mask, src):
    res = _f(res).copy()
    sel = _f(mask).reshape(res.shape) != 0
    res[sel] = _f(src).reshape(-1)[:int(sel.sum())]
    return res
