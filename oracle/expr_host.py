"""CPU evaluation of an apply/map/map2 expression string: TEST INFRASTRUCTURE.

The statement is compiled for the host with gcc in fp32 (contraction off) and
run over dense arrays.  The text transformation is written here independently
of the library's: ``x``/``y``/``z`` become the operands the reference assigns
them (src/lib/THClTensorMathPointwise.cpp:79-146) and unsuffixed floating
literals become fp32, the type an fp32-only OpenCL C device gives them.
Expressions made of + - * / sqrt are correctly rounded on both sides and
compare bit for bit; transcendental functions compare within the reference
tests' own tolerance (src/test/unit_tensor.lua:73-93).

Pinned by tests/test_oracle.py (no GPU needed): ``rewrite`` against the
reference's substitutions on its own test strings in both spellings, names
that contain x/y/z, and literal typing; ``evaluate`` against IEEE fp32
arithmetic written one rounding at a time with numpy (two roundings told
from a fused multiply-add, fp32 literals told from double ones, operand
binding, the prelude functions) and the transcendental statements within one
unit of the last place of fp64-then-round.
"""
import ctypes as C
import hashlib
import os
import re
import subprocess
import tempfile

import numpy as np

_PRELUDE = r"""
#include <math.h>
#define max(a, b) ((a) < (b) ? (b) : (a))
#define min(a, b) ((b) < (a) ? (b) : (a))
#define sqrt sqrtf
#define exp expf
#define log logf
#define fabs fabsf
#define tanh tanhf
#define pow powf
#define floor floorf
#define ceil ceilf
#define sin sinf
#define cos cosf
static inline float pown(float x, int n) { return powf(x, (float)n); }
static inline float clamp(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }
static inline float sign(float x) { return (float)((x > 0.0f) - (x < 0.0f)); }
"""

_cache = {}
_dir = None


def rewrite(expr: str, ntensors: int) -> str:
    names = {"x": "(*out)"}
    if ntensors >= 2:
        names["y"] = "(*in1)"
    if ntensors >= 3:
        names["z"] = "(*in2)"
    expr = re.sub(r"\b([xyz])\b", lambda m: names.get(m.group(1), m.group(1)), expr)
    # 1.5  2.  .5  1e-3  -> fp32 literals (leave integers and already suffixed ones alone)
    lit = re.compile(r"(?<![\w.])((?:\d+\.\d*|\.\d+)(?:[eE][+-]?\d+)?|\d+[eE][+-]?\d+)(?![\w.])")
    return lit.sub(lambda m: m.group(1) + "f", expr)


def compile_expr(expr: str, ntensors: int):
    global _dir
    key = (expr, ntensors)
    if key in _cache:
        return _cache[key]
    if _dir is None:
        _dir = tempfile.mkdtemp(prefix="thcl_oracle_expr_")
    body = rewrite(expr, ntensors)
    src = _PRELUDE + """
void run(float *o, const float *a, const float *b, long n) {
  for (long i = 0; i < n; i++) {
    float ov = o[i], av = a ? a[i] : 0.0f, bv = b ? b[i] : 0.0f;
    float *out = &ov, *in1 = &av, *in2 = &bv;
    (void)in1; (void)in2;
    %s;
    o[i] = ov;
  }
}
""" % body
    tag = hashlib.sha1(src.encode()).hexdigest()[:16]
    cpath, sopath = os.path.join(_dir, tag + ".c"), os.path.join(_dir, tag + ".so")
    with open(cpath, "w") as f:
        f.write(src)
    subprocess.check_call(["gcc", "-O2", "-ffp-contract=off", "-fno-fast-math", "-shared", "-fPIC", "-o", sopath,
                           cpath, "-lm"])
    fn = C.CDLL(sopath).run
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_long]
    fn.restype = None
    _cache[key] = fn
    return fn


def evaluate(expr: str, out: np.ndarray, in1: np.ndarray = None, in2: np.ndarray = None) -> np.ndarray:
    """Applies the statement element-wise to dense fp32 arrays; returns the new ``out``."""
    n = 1 + (in1 is not None) + (in2 is not None)
    fn = compile_expr(expr, n)
    o = np.ascontiguousarray(out, dtype=np.float32).copy()
    a = np.ascontiguousarray(in1, dtype=np.float32) if in1 is not None else None
    b = np.ascontiguousarray(in2, dtype=np.float32) if in2 is not None else None
    fn(o.ctypes.data, a.ctypes.data if a is not None else None, b.ctypes.data if b is not None else None, o.size)
    return o
