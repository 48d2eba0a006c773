"""Torch7's text form of tensors and storages (``tostring(clTensor)``; in the reference the Lua
binding copies the tensor to the host and lets Torch7's ``Tensor.__tostring__`` format it).

The rules are Torch7's (``torch/Tensor.lua``: one common number format per tensor, chosen from
the magnitudes present; integer-valued data print as integers).  The reference's tests hold the
expected text for vectors, matrices and storages of small integers and of 4-decimal fractions
(src/test/unit_tensor.lua:164-199, src/test/unit_storage.lua:24-58); the scaled, exponent and
N-d slice forms follow the same source but have no expected text in the reference.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np


def _c_format(fmt: str, value: float) -> str:
    if fmt.endswith("d"):
        if math.isnan(value) or math.isinf(value):      # Lua's %d of these is platform noise; print them as C's %f would
            return ("%" + fmt[1:-1] + "s") % ("nan" if math.isnan(value) else ("inf" if value > 0 else "-inf"))
        return fmt % int(value)
    return fmt % value


def _print_format(values: np.ndarray) -> Tuple[str, Optional[float], int]:
    """(format, scale or None, field width) for a flat array of doubles."""
    if values.size == 0:
        return "", None, 0
    with np.errstate(invalid="ignore"):
        int_mode = bool(np.all(values == np.ceil(values)))
    mags = np.abs(values)
    finite = mags[np.isfinite(mags)]
    lo = float(finite.min()) if finite.size else 0.0
    hi = float(finite.max()) if finite.size else 0.0
    exp_min = math.floor(math.log10(lo)) + 1 if lo != 0 else 1
    exp_max = math.floor(math.log10(hi)) + 1 if hi != 0 else 1
    scale = None
    if int_mode:
        if exp_max > 9:
            fmt, width = "%11.4e", 11
        else:
            width = exp_max + 1
            fmt = "%%%dd" % width
    elif exp_max - exp_min > 4:
        width = 11 + (1 if abs(exp_max) > 99 or abs(exp_min) > 99 else 0)
        fmt = "%%%d.4e" % width
    elif exp_max > 5 or exp_max < 0:
        width = 7
        fmt = "%7.4f"
        scale = math.pow(10, exp_max - 1)
    else:
        width = 7 if exp_max == 0 else exp_max + 6
        fmt = "%%%d.4f" % width
    if scale == 1:
        scale = None
    return fmt, scale, width


def _matrix(m: np.ndarray, fmt: str, scale: Optional[float], width: int, indent: str = "") -> str:
    scale_v = scale or 1.0
    out = [indent]
    rows, cols = m.shape
    per_line = (80 - len(indent)) // (width + 1)
    first = 0
    while first < cols:
        last = min(first + per_line, cols)
        if per_line < cols:
            if first != 0:
                out.append("\n")
            out.append("Columns %d to %d\n%s" % (first + 1, last, indent))
        if scale_v != 1:
            out.append("%g *\n %s" % (scale_v, indent))
        for r in range(rows):
            for c in range(first, last):
                out.append(_c_format(fmt, float(m[r, c]) / scale_v))
                if c == last - 1:
                    out.append("\n")
                    if r != rows - 1:
                        out.append(indent + (" " if scale_v != 1 else ""))
                else:
                    out.append(" ")
        first = last
    return "".join(out)


def tensor_tostring(values: np.ndarray, typename: str = "torch.ClTensor") -> str:
    """``tostring(tensor)`` for a host copy of the tensor's elements."""
    a = np.asarray(values, dtype=np.float64)
    if a.ndim == 0 or a.size == 0 and a.ndim <= 1:
        return "[%s with no dimension]\n" % typename
    fmt, scale, width = _print_format(a.reshape(-1))
    size_text = "x".join(str(s) for s in a.shape)
    if a.ndim == 1:
        lines = []
        if scale:
            lines.append("%g *\n" % scale)
        for v in a:
            lines.append(_c_format(fmt, float(v) / (scale or 1.0)) + "\n")
        return "".join(lines) + "[%s of size %d]\n" % (typename, a.shape[0])
    if a.ndim == 2:
        return _matrix(a, fmt, scale, width) + "[%s of size %s]\n" % (typename, size_text)
    # N-d: one matrix per setting of the leading indices, the first index running fastest
    lead = a.shape[:-2]
    out = []
    count = int(np.prod(lead))
    for n in range(count):
        idx, rest = [], n
        for s in lead:
            idx.append(rest % s)
            rest //= s
        if out:
            out.append("\n")
        out.append("(" + "".join("%d," % (i + 1) for i in idx) + ".,.) = \n")
        out.append(_matrix(a[tuple(idx)], fmt, scale, width, " "))
    return "".join(out) + "[%s of size %s]\n" % (typename, size_text)


def storage_tostring(values: np.ndarray, typename: str = "torch.ClStorage") -> str:
    """``tostring(storage)``: one element per line in the storage's common format."""
    a = np.asarray(values, dtype=np.float64).reshape(-1)
    fmt, scale, _ = _print_format(a)
    lines = []
    if scale:
        lines.append("%g *\n" % scale)
    for v in a:
        lines.append(_c_format(fmt, float(v) / (scale or 1.0)) + "\n")
    return "".join(lines) + "[%s of size %d]\n" % (typename, a.size)
