"""CPU-side checks of the shipped library: it loads, exports what the headers
declare, never routes through the oracle, and its host logic (layout rules,
index division, expression rewrite + run-time compile) is right.  No kernel is
launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle
from cltorch_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MAXD = 25


@pytest.fixture(scope="module")
def lib(hooks_lib):
    L = hooks_lib                       # the library's objects plus the test-only entry points
    for name, (res, args) in _lib.declared_symbols().items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    L.thcl_dbg_divide.restype = C.c_uint
    L.thcl_dbg_divide.argtypes = [C.c_uint, C.c_long]
    L.thcl_dbg_rewrite_expr.restype = C.c_int
    L.thcl_dbg_rewrite_expr.argtypes = [C.c_char_p, C.c_int, C.c_char_p, C.c_size_t]
    L.thcl_dbg_compile_expr.restype = C.c_int
    L.thcl_dbg_compile_expr.argtypes = [C.c_char_p, C.c_int, C.c_char_p, C.POINTER(C.c_size_t)]
    return L


def test_library_exports_every_declared_symbol():
    decls = _lib.declared_symbols()
    assert len(decls) > 120
    L = C.CDLL(_lib.LIB_PATH)
    missing = [n for n in decls if not hasattr(L, n)]
    assert not missing, missing
    for must in ("THClTensor_cadd", "THClTensor_cmul", "THClTensor_div", "THClTensor_div_gpu", "THClTensor_apply",
                 "THClTensor_map", "THClTensor_map2", "THClTensor_copy", "THClTensor_sumall", "THClTensor_sumall_gpu",
                 "THClTensor_maxall", "THClTensor_minall", "THClTensor_sum", "THClTensor_max", "THClTensor_min",
                 "THClTensor_addmm", "THClBlas_gemm", "THClTensor_as_float", "thcl_rt_kernel_get", "thcl_rt_launch"):
        assert must in decls, must


def test_library_exports_only_what_the_headers_declare():
    """Built with hidden visibility: the dynamic symbol table holds the declared entry points and no test hook,
    internal C++ function or kernel stub."""
    import subprocess
    decls = set(_lib.declared_symbols())
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    extra = sorted(n for n in exported - decls if not n.startswith(("_init", "_fini", "__bss", "_edata", "_end", "__hip_")))
    assert not extra, extra[:20]
    assert not any("dbg" in n for n in exported)


def test_library_defines_every_function_the_reference_library_defines():
    """tests/golden/reference_defined_exports.json lists the functions the reference declares THCL_API in a header and
    defines in a .cpp file of its tensor library (written by tests/golden/make_reference_exports.py from the
    reference's text): a binding linked from the reference's unchanged sources may name any of them, so the library
    that takes its place has to resolve them all -- also the ones the reference defines only to raise an error."""
    import json
    import subprocess
    names = json.load(open(os.path.join(ROOT, "tests", "golden", "reference_defined_exports.json")))["names"]
    assert len(names) > 150
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    missing = [n for n in names if n not in exported]
    assert not missing, missing


def test_reference_stubs_report_the_reference_messages(lib):
    """The entry points the reference defines only to raise (src/lib/THClStorage.cpp:142-200, THClStorageCopy.cpp:27-32,
    THClBlas.cpp:67-147,451-470, THClTensorMathBlas.cpp:279-380) raise here with the same text, before any device
    is touched."""
    lib.THClLastError.restype = C.c_char_p
    f = C.c_float
    calls = {
        "THClStorage_newWithSize1": (None, 0, f(1)), "THClStorage_newWithSize2": (None, 0, f(1), f(2)),
        "THClStorage_newWithSize3": (None, 0, f(1), f(2), f(3)), "THClStorage_newWithSize4": (None, 0, f(1), f(2), f(3), f(4)),
        "THClStorage_newWithMapping": (None, 0, b"file", 4, 0), "THClStorage_newWithData": (None, 0, None, 4),
        "THClStorage_copyCl": (None, None, None),
    }
    for name, args in calls.items():
        r = getattr(lib, name)(*args)
        assert not r
        assert lib.THClLastError() == b"not available yet for THClStorage", name
    blas = {
        "THClBlas_swap": (None, 4, None, 1, None, 1), "THClBlas_scal": (None, 4, f(2), None, 1),
        "THClBlas_copy": (None, 4, None, 1, None, 1), "THClBlas_axpy": (None, 4, f(2), None, 1, None, 1),
        "THClBlas_gemmBatched": (None, b"n", b"n", 2, 2, 2, f(1), None, 2, None, 2, f(0), None, 2, 1),
        "THClTensor_baddbmm": (None, None, f(1), None, f(1), None, None),
    }
    for name, args in blas.items():
        getattr(lib, name)(*args)
        assert lib.THClLastError() == b"Not implemented", name


def test_product_never_touches_the_oracle():
    pat = re.compile(r"\boracle\b")
    for base, _, files in os.walk(os.path.join(ROOT, "cltorch_amd")):
        if os.path.basename(base) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h", ".inc")):
                text = open(os.path.join(base, f)).read()
                assert not pat.search(text), f"{f} mentions the oracle"
    for f in os.listdir(os.path.join(ROOT, "include")):
        assert not pat.search(open(os.path.join(ROOT, "include", f)).read())


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libthcl_hip.so")
    with pytest.raises(_lib.LibraryMissing):
        _lib.load()


def test_no_device_is_an_error_not_a_fallback():
    L = _lib.load()
    if L.thcl_rt_device_count() > 0:
        pytest.skip("a GPU is visible")
    buf = C.create_string_buffer(256)
    st = C.cast(buf, C.c_void_p)
    L.THCl_initializeState(st)
    L.THClInit(st)
    err = L.THClLastError()
    assert err and b"no HIP device" in err


def test_multiply_shift_division_is_exact(lib):
    rng = np.random.RandomState(0)
    divisors = [1, 2, 3, 4, 5, 7, 10, 63, 64, 65, 127, 128, 255, 256, 1000, 4096, 16384, 65535, 65536, 65537,
                131072, 2 ** 25, 2 ** 26 - 1, 2 ** 30, 2 ** 31 - 1] + [int(v) for v in rng.randint(1, 2 ** 31 - 1, 40)]
    for d in divisors:
        ns = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 2 ** 31 - 1, 2 ** 31 - 2] + [int(v) for v in rng.randint(0, 2 ** 31 - 1, 200)]
        for n in ns:
            if 0 <= n < 2 ** 31:
                assert lib.thcl_dbg_divide(n, d) == n // d, (n, d)


def _arr(vals, n=MAXD):
    a = (C.c_long * n)()
    for i, v in enumerate(vals):
        a[i] = v
    return a


def test_collapse_matches_oracle_rule(lib):
    rng = np.random.RandomState(1)
    for _ in range(400):
        nd = rng.randint(1, 6)
        sizes = [int(rng.choice([1, 1, 2, 3, 4, 6])) for _ in range(nd)]
        strides = [int(rng.choice([0, 1, 2, 3, 4, 6, 8, 12, 24])) for _ in range(nd)]
        rd = int(rng.randint(-1, nd))
        osz, ost = (C.c_long * MAXD)(), (C.c_long * MAXD)()
        k = lib.thcl_dbg_collapse(nd, _arr(sizes), _arr(strides), rd, osz, ost)
        want = oracle.collapse(sizes, strides, rd)
        assert (list(osz[:k]), list(ost[:k])) == want
        assert bool(lib.thcl_dbg_overlapping(nd, _arr(sizes), _arr(strides))) == oracle.overlapping(sizes, strides)


def _offsets(sizes, strides):
    idx = np.indices(sizes).reshape(len(sizes), -1)
    return (idx * np.array(strides).reshape(-1, 1)).sum(axis=0)


def test_joint_collapse_pairs_the_same_elements(lib):
    """Walking the joint layout must visit exactly the (offset0, offset1, ...) tuples
    that walking the operands in logical order visits -- in any order."""
    rng = np.random.RandomState(2)
    for _ in range(300):
        nd = rng.randint(1, 5)
        n = rng.randint(1, 4)
        sizes = [int(rng.choice([1, 2, 3, 4, 5])) for _ in range(nd)]
        all_strides = []
        for i in range(n):
            perm = rng.permutation(nd)
            st, z = [0] * nd, 1
            for d in perm:                       # dense in a random dim order, sometimes with gaps
                st[d] = z
                z *= sizes[d] * int(rng.choice([1, 1, 2]))
            if i > 0 and rng.rand() < 0.2:
                st[int(rng.randint(nd))] = 0     # broadcast input
            all_strides.append(st)
        szs = (C.c_long * (3 * MAXD))()
        sts = (C.c_long * (3 * MAXD))()
        for i in range(n):
            for d in range(nd):
                szs[i * MAXD + d] = sizes[d]
                sts[i * MAXD + d] = all_strides[i][d]
        osz, ost = (C.c_long * MAXD)(), (C.c_long * (3 * MAXD))()
        k = lib.thcl_dbg_joint_collapse(n, (C.c_int * 3)(*([nd] * n + [0] * (3 - n))), szs, sts, osz, ost)
        assert k >= 1
        jsz = list(osz[:k])
        want = set(zip(*[_offsets(sizes, all_strides[i]).tolist() for i in range(n)]))
        got = set(zip(*[_offsets(jsz, [ost[i * MAXD + d] for d in range(k)]).tolist() for i in range(n)]))
        assert got == want
        assert int(np.prod(jsz)) == int(np.prod(sizes))


def test_joint_collapse_makes_identically_transposed_views_dense(lib):
    szs, sts = (C.c_long * (3 * MAXD))(), (C.c_long * (3 * MAXD))()
    for i in range(2):
        for d, (s, t) in enumerate(zip((256, 512, 512), (1, 256, 131072))):
            szs[i * MAXD + d], sts[i * MAXD + d] = s, t
    osz, ost = (C.c_long * MAXD)(), (C.c_long * (3 * MAXD))()
    k = lib.thcl_dbg_joint_collapse(2, (C.c_int * 3)(3, 3, 0), szs, sts, osz, ost)
    assert k == 1 and osz[0] == 2 ** 26 and ost[0] == 1 and ost[MAXD] == 1
    # different shapes with equal element counts are not joint-collapsible
    szs[MAXD + 0], szs[MAXD + 1], szs[MAXD + 2] = 512, 256, 512
    assert lib.thcl_dbg_joint_collapse(2, (C.c_int * 3)(3, 3, 0), szs, sts, osz, ost) == -1


def _rewrite(lib, expr, n):
    buf = C.create_string_buffer(4096)
    r = lib.thcl_dbg_rewrite_expr(expr.encode(), n, buf, 4096)
    assert r >= 0
    return buf.value.decode()


def test_expression_rewrite(lib):
    # the two spellings the reference's tests use (src/test/unit_tensor.lua:583-635)
    assert _rewrite(lib, "x = sqrt(x + 3) + exp(x)", 1) == "(*out) = sqrt((*out) + 3) + exp((*out))"
    assert _rewrite(lib, "*out = sqrt(*out + 3) + exp(*out)", 1) == "*out = sqrt(*out + 3) + exp(*out)"
    assert _rewrite(lib, "x = sqrt(x * x + y * y + z + 3 + exp(z))", 3) == \
        "(*out) = sqrt((*out) * (*out) + (*in1) * (*in1) + (*in2) + 3 + exp((*in2)))"
    # y / z are only operands when the call has that many tensors (src/lib/THClTensorMathPointwise.cpp:79-146)
    assert _rewrite(lib, "x = y + z", 1) == "(*out) = y + z"
    assert _rewrite(lib, "x = y + z", 2) == "(*out) = (*in1) + z"
    # identifiers containing x/y/z survive (the reference only shields exp and max)
    assert _rewrite(lib, "x = max(x, y) + hypot(x, y) + copysign(x, z)", 3) == \
        "(*out) = max((*out), (*in1)) + hypot((*out), (*in1)) + copysign((*out), (*in2))"
    # floating literals become fp32, integer literals and suffixed ones stay
    assert _rewrite(lib, "x = 1000*x + 0.5 + 1e-3 + 2. + .25 + 3.5f + 7", 1) == \
        "(*out) = 1000*(*out) + 0.5f + 1e-3f + 2.f + .25f + 3.5f + 7"


@pytest.mark.parametrize("expr,n", [
    ("x = sqrt(1000*x*x + y*10 + z*z)", 3),
    ("x = 1000*x + y*10", 2),
    ("*out = sqrt(*out * *out + *in1 * *in1 + 3 + exp(*in1))", 2),
    ("x = clamp(x, -0.5, 0.5) + pown(x, 3) + sign(x) + fmax(x, 0.1)", 1),
])
def test_expressions_compile_for_gfx950(lib, expr, n):
    size = C.c_size_t(0)
    rc = lib.thcl_dbg_compile_expr(expr.encode(), n, b"gfx950", C.byref(size))
    assert rc == 0, lib.thcl_rt_error().decode()
    assert size.value > 1000


def test_bad_expression_reports_compiler_log(lib):
    size = C.c_size_t(0)
    rc = lib.thcl_dbg_compile_expr(b"x = this is not C", 1, b"gfx950", C.byref(size))
    assert rc != 0
    assert b"error" in lib.thcl_rt_error()


# ------------------------------------------------------------ kernel planning ---
KINDS = {0: "dense128", 1: "dense32", 2: "joint128", 3: "joint32", 4: "generic", 5: "tiled", 6: "nothing", -1: "rejected"}


def _plan(lib, views, misalign=None):
    """views: list of (sizes, strides, offset).  Returns (kind name, grid)."""
    n = len(views)
    lib.thcl_dbg_plan_kind.restype = C.c_int
    szs, sts = (C.c_long * (3 * MAXD))(), (C.c_long * (3 * MAXD))()
    nd, off, mis = (C.c_int * 3)(), (C.c_long * 3)(), (C.c_int * 3)()
    for i, (sz, st, o) in enumerate(views):
        nd[i], off[i] = len(sz), o
        mis[i] = (misalign or [0] * n)[i]
        for d in range(len(sz)):
            szs[i * MAXD + d], sts[i * MAXD + d] = sz[d], st[d]
    grid = C.c_uint(0)
    k = lib.thcl_dbg_plan_kind(n, nd, szs, sts, off, mis, C.byref(grid))
    return KINDS[k], grid.value


def test_planner_picks_the_kernel_family_for_each_layout(lib):
    dense = ((512, 512, 256), (131072, 256, 1), 0)
    assert _plan(lib, [dense, dense]) == ("dense128", 2 ** 26 // 4 // 64)         # one-wave blocks, 4 floats per lane
    assert _plan(lib, [dense, dense, dense]) == ("dense128", 2 ** 26 // 2 // 64)  # three operands: 2 floats per lane
    assert _plan(lib, [dense]) == ("dense128", 2 ** 26 // 4 // 256)
    assert _plan(lib, [dense, dense], [0, 4])[0] == "dense32"                       # one operand 4 bytes off
    assert _plan(lib, [((100,), (1,), 1), ((100,), (1,), 0)])[0] == "dense32"       # odd element offset
    tr = ((256, 512, 512), (1, 256, 131072), 0)
    assert _plan(lib, [tr, tr])[0] == "dense128"                                    # identically transposed: dense walk
    dst = ((256, 512, 512), (262144, 512, 1), 0)
    kind, grid = _plan(lib, [dst, tr])
    assert kind == "tiled" and grid == 512 * (512 // 64) * (256 // 256)             # 64 x 256 tiles, 512 outer slices
    sq = _plan(lib, [((8192, 8192), (8192, 1), 0), ((8192, 8192), (1, 8192), 0)])
    assert sq == ("tiled", (8192 // 128) ** 2)                                      # plain 2-d transpose: 128 x 128 tiles
    # element counts: dense walks index with 64 bits, strided walks refuse what 32-bit indices cannot reach
    n = (1 << 31) + 4096
    assert _plan(lib, [((n,), (1,), 0), ((n,), (1,), 0)])[0] == "dense128"
    assert _plan(lib, [((n // 2, 2), (1, n // 2), 0)])[0] == "dense128"               # a transposed walk that is dense after sorting dims
    assert _plan(lib, [((n,), (2,), 0)])[0] == "rejected"                              # gapped: 32-bit linear index would overflow
    assert _plan(lib, [((n // 2,), (2,), 0)])[0] in ("joint32", "joint128")
    # a rank-1 update: vectors expanded with stride 0 ride the vector kernel, not the transposing tiles
    outer = _plan(lib, [((4096, 4096), (4096, 1), 0), ((4096, 4096), (1, 0), 0), ((4096, 4096), (0, 1), 0)])
    assert outer[0] == "joint128"
    thin = _plan(lib, [((1024, 64, 1024), (65536, 1024, 1), 0), ((1024, 64, 1024), (65536, 1, 64), 0)])
    assert thin == ("tiled", 1024 * (1024 // 256) * (64 // 64))                     # dim B of 64: 256 x 64 tiles waste nothing
    assert _plan(lib, [tr, dst])[0] == "tiled"                                      # scatter into the transposed view
    s2 = ((512, 512, 128), (131072, 256, 2), 0)
    assert _plan(lib, [s2, s2])[0] == "joint32"
    nar = ((512, 512, 128), (131072, 256, 1), 64)
    assert _plan(lib, [nar, nar])[0] == "joint128"
    assert _plan(lib, [nar, ((512, 512, 128), (131072, 256, 1), 65)])[0] == "joint32"   # rows not 16-byte aligned
    assert _plan(lib, [((30, 28), (28, 1), 0), ((28, 30), (1, 56), 0)])[0] == "generic"  # shapes differ
    assert _plan(lib, [((4, 5), (5, 1), 0), ((21,), (1,), 0)])[0] == "rejected"     # element counts differ
    assert _plan(lib, [((3, 4), (4, 1), 0)])[0] == "dense128"
    # tiny transposed operands are not worth a tile
    assert _plan(lib, [((8, 8), (8, 1), 0), ((8, 8), (1, 8), 0)])[0] == "joint32"


def test_user_kernel_renders_and_compiles_for_gfx950(lib):
    """The reference's README kernel (README.md:135-160) through THClKernel_new, compiled offline."""
    lib.THClKernel_new.restype = C.c_void_p
    lib.THClKernel_new.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_char_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.THClKernel_getRenderedKernel.restype = C.c_char_p
    lib.THClKernel_getRenderedKernel.argtypes = [C.c_void_p]
    lib.THClKernel_compileCheck.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_size_t)]
    lib.THClKernel_free.argtypes = [C.c_void_p, C.c_void_p]
    names = (C.c_char_p * 3)(b"input", b"nElements", b"output")
    types, dirs = (C.c_int * 3)(2, 0, 2), (C.c_int * 3)(0, 0, 1)
    src = b"int linearId = get_global_id(0); if(linearId < nElements) { output_data[linearId] = input_data[linearId] + 3.0f; }"
    k = lib.THClKernel_new(None, None, src, None, 3, names, types, dirs)
    assert k
    text = lib.THClKernel_getRenderedKernel(k).decode()
    assert "void user_kernel(" in text and "const float *input_data" in text and "int nElements" in text
    size = C.c_size_t(0)
    assert lib.THClKernel_compileCheck(k, b"gfx950", C.byref(size)) == 0, lib.thcl_rt_error().decode()
    assert size.value > 1000
    lib.THClKernel_free(None, k)


def test_gemm_tile_choice(lib):
    """The tile comes from a model of the launch: the kernel's rate, whole rounds of tiles per CU, the tiles' area
    outside the matrix, blocks per CU, K slicing.  Known outcomes on 256 CUs, each confirmed by measurement."""
    def tile(m, n, k, cus=256):
        bm, bn, ks, kc, tt, ts = (C.c_int(0) for _ in range(6))
        lib.thcl_dbg_gemm_plan(C.c_long(m), C.c_long(n), C.c_long(k), C.c_int(cus), C.byref(bm), C.byref(bn), C.byref(ks), C.byref(kc),
                               C.byref(tt), C.byref(ts))
        return bm.value, bn.value
    assert tile(8192, 8192, 8192) == (128, 128) and tile(4096, 4096, 4096) == (128, 128) and tile(6144, 6144, 6144) == (128, 128)
    # the skinny configuration after the row-major swap, when the streaming kernel cannot take it (calls in a row: 64x64
    # tiles in 2 slices 90 us, 128x64 tiles in 4 slices 94)
    assert tile(16384, 64, 4096) == (64, 64)
    # a few tiles more than a whole number per CU: the surplus tiles share their K, so the large tile keeps its rate
    # (4608^3: 135 TFLOP/s in 128x64 tiles -> 147; 3072^3: 123 in 64x64 tiles -> 145)
    assert tile(4608, 4608, 4608) == (128, 128) and tile(5120, 5120, 5120) == (128, 128) and tile(3072, 3072, 3072) == (128, 128)
    assert tile(2560, 2560, 2560) == (64, 128)     # 400 tiles of 128x128 leave more than half the CUs a second tile; 800 of 64x128 leave 32
    assert tile(2048, 2048, 2048) == (64, 64) and tile(1024, 1024, 1024) == (64, 64)
    assert tile(100, 100, 100) == (64, 64)
    # ragged sizes: every tile shape has edges, the larger tiles' edge kernels keep the higher rate
    assert tile(6000, 6000, 2000) == (128, 64)     # 4418 tiles, the last 66 share their K (135 TFLOP/s in 128x128 tiles, 139)
    # 960 tiles of 128x128 are 3.75 per CU; 1920 of 128x64 are 7.5 with the last 104 sharing their K (125 -> 134 TFLOP/s)
    assert tile(3000, 5000, 7000) == (128, 64)
    # 63 x 64 rows and columns: whole 64-wide tiles (123 x 0.97 for the last round) lose to 128-wide ones with edges (128 x 0.97 of area)
    assert tile(4032, 4032, 4096) == (128, 128)
    # a side of at most 32: thin tiles halve the padding of a 64-wide tile; they never stand for wider products
    assert tile(16384, 16, 16384) == (128, 32) and tile(32, 4096, 1024) == (32, 128) and tile(4096, 32, 4096) == (128, 32)
    assert tile(16384, 33, 4096)[1] == 64 and tile(40, 4096, 4096)[0] == 64
    assert tile(20, 20, 64) == (64, 64)


def test_gemm_k_slicing(lib):
    """K is sliced when there are too few tiles for the chip: below one tile per CU from K = 1024 up, below
    two tiles per CU from K = 2048 up, below half a tile per CU from K = 512 up; slices are multiples of the K slab (16)
    and at least 256 long, or 128 where slices of 256 would leave CUs without a block."""
    def plan(m, n, k, cus=256):
        bm, bn, ks, kc, tt, ts = (C.c_int(0) for _ in range(6))
        lib.thcl_dbg_gemm_plan(C.c_long(m), C.c_long(n), C.c_long(k), C.c_int(cus), C.byref(bm), C.byref(bn),
                               C.byref(ks), C.byref(kc), C.byref(tt), C.byref(ts))
        return bm.value, bn.value, ks.value, kc.value
    assert plan(8192, 8192, 8192) == (128, 128, 1, 8192)
    assert plan(16384, 64, 4096) == (64, 64, 2, 2048)            # skinny: 256 tiles on 256 CUs, a long K
    assert plan(2048, 512, 4096) == (64, 128, 4, 1024)           # 128 tiles, long K: the same 512 blocks as 256 tiles in 2 slices, at the larger tile's rate
    assert plan(1024, 1024, 1024) == (64, 64, 1, 1024)           # 256 tiles but K too short to pay for a second pass
    assert plan(64, 64, 100000)[2] == 368                        # one tile: as many slices of at least 256 as fit
    assert plan(32, 32, 1 << 20)[2] == 512                       # capped
    assert plan(128, 128, 400)[2:] == (1, 400)                   # K below 512 is never sliced
    assert plan(128, 128, 1000)[2:] == (7, 144)                  # very few tiles: slices down to 128 (23 -> 9.6 us)
    assert plan(512, 512, 512)[2:] == (4, 128)                   # 64 tiles: 13.2 -> 10.6 us
    assert plan(256, 1024, 1024)[2:] == (4, 256)                 # 64 tiles, and slices of 256 already give every CU a block
    # several tiles per CU and a few left over (at most half the CUs): those are each shared by floor(CUs / leftover)
    # blocks along K, at most 16, slices of at least 256
    def tail(m, n, k, cus=256):
        v = [C.c_int(0) for _ in range(6)]
        lib.thcl_dbg_gemm_plan(C.c_long(m), C.c_long(n), C.c_long(k), C.c_int(cus), *[C.byref(x) for x in v])
        return v[4].value, v[5].value
    assert tail(3072, 3072, 3072) == (64, 4) and tail(4608, 4608, 4608) == (16, 16) and tail(4100, 4100, 4100) == (65, 3)
    assert tail(3072, 3072, 600) == (128, 2) and tail(3072, 3072, 500) == (0, 1)     # 1152 tiles of 128x64; K too short to share
    assert tail(8192, 8192, 8192) == (0, 1) and tail(4095, 4095, 4095) == (0, 1)     # whole numbers of tiles per CU
    assert tail(4096, 6016, 4096) == (0, 1)                                          # 1504 tiles: 224 left over, more than half the CUs
    assert tail(4096, 7680, 4096) == (128, 2)                                        # 1920 tiles: exactly half the CUs left over
    assert tail(64, 64, 100000) == (0, 1)                                            # sliced over the whole grid instead
    for k in (1024, 1040, 3000, 5555):
        _, _, ks, kc = plan(64, 64, k)
        assert kc % 16 == 0 and (ks - 1) * kc < k <= ks * kc and (ks == 1 or kc >= 128)


def test_torch7_file_framing_known_bytes():
    """The bytes written for a 2 x 3 tensor at offset 1 of a 7-element storage, assembled by hand from
    the field order of src/torch/generic/Tensor.cpp:1290-1304 and Storage.cpp:255-266 inside Torch7's
    object framing; then the reader's error paths."""
    import struct
    from cltorch_amd import serialize as S
    data = np.array([9, 1, 2, 3, 4, 5, 6], dtype=np.float32)
    want = b"".join([
        struct.pack("<ii", 4, 1), struct.pack("<i", 3), b"V 1", struct.pack("<i", 14), b"torch.ClTensor",
        struct.pack("<i", 2), struct.pack("<qq", 2, 3), struct.pack("<qq", 3, 1), struct.pack("<q", 2),
        struct.pack("<ii", 4, 2), struct.pack("<i", 3), b"V 1", struct.pack("<i", 15), b"torch.ClStorage",
        struct.pack("<q", 7), data.tobytes()])
    got = S.encode_tensor([2, 3], [3, 1], 1, data)
    assert got == want
    sizes, strides, off, storage, tclass, sclass = S.decode_tensor(got)
    assert (sizes, strides, off, tclass, sclass) == ([2, 3], [3, 1], 1, "torch.ClTensor", "torch.ClStorage")
    assert np.array_equal(storage, data)
    # an empty tensor: the header's dimension field is -1 and the storage is nil, as the reference writes it
    # (src/lib/THClTensor.cpp:635, src/torch/generic/Tensor.cpp:1296-1310)
    empty = S.encode_tensor([], [], 0, None)
    assert empty == b"".join([struct.pack("<ii", 4, 1), struct.pack("<i", 3), b"V 1", struct.pack("<i", 14), b"torch.ClTensor",
                              struct.pack("<i", -1), struct.pack("<q", 1), struct.pack("<i", 0)])
    assert S.decode_tensor(empty)[:4] == ([], [], 0, None)
    # a point tensor: no dimensions, but a storage of one value
    point = S.encode_tensor([], [], 0, np.array([2.5], dtype=np.float32))
    assert point == b"".join([struct.pack("<ii", 4, 1), struct.pack("<i", 3), b"V 1", struct.pack("<i", 14), b"torch.ClTensor",
                              struct.pack("<i", 0), struct.pack("<q", 1),
                              struct.pack("<ii", 4, 2), struct.pack("<i", 3), b"V 1", struct.pack("<i", 15), b"torch.ClStorage",
                              struct.pack("<q", 1), struct.pack("<f", 2.5)])
    sizes, strides, off, storage, _, _ = S.decode_tensor(point)
    assert (sizes, strides, off) == ([], [], 0) and storage.tolist() == [2.5]
    # and a 1-d tensor over the whole of its storage
    one = S.encode_tensor([3], [1], 0, np.array([1, 2, 3], dtype=np.float32))
    assert S.decode_tensor(one)[:3] == ([3], [1], 0) and S.decode_tensor(one)[3].tolist() == [1, 2, 3]
    for bad in (got[:-2], got[:40], got.replace(b"torch.ClTensor", b"torch.XxTensor"), struct.pack("<ii", 3, 1) + got[8:]):
        with pytest.raises(ValueError):
            S.decode_tensor(bad)


def test_text_form_matches_the_reference_expected_strings():
    """tostring of tensors and storages against every expected string the reference's tests hold."""
    import json
    from cltorch_amd.printing import storage_tostring, tensor_tostring
    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))["tostring"]
    for case in gold["tensors"]:
        assert tensor_tostring(np.array(case["values"], dtype=np.float32), case["type"]) == case["text"], case
    for case in gold["storages"]:
        assert storage_tostring(np.array(case["values"], dtype=np.float32), case["type"]) == case["text"], case
    # forms without an expected string in the reference: structure only
    wide = tensor_tostring(np.arange(60, dtype=np.float32).reshape(2, 30))
    assert wide.startswith("Columns 1 to 20\n") and "\nColumns 21 to 30\n" in wide and wide.endswith("[torch.ClTensor of size 2x30]\n")
    nd = tensor_tostring(np.zeros((2, 2, 2), dtype=np.float32))
    assert nd.startswith("(1,.,.) = \n  0  0\n  0  0\n\n(2,.,.) = \n") and nd.endswith("[torch.ClTensor of size 2x2x2]\n")
    assert tensor_tostring(np.array([1e-3, 5.0, 123456.0])).splitlines()[0] == " 1.0000e-03"
    assert tensor_tostring(np.zeros(())) == "[torch.ClTensor with no dimension]\n"


def test_public_structs_keep_the_reference_field_layout(tmp_path):
    """LuaJIT code reads THClStorage / THClTensor fields directly (src/FFI.lua:6-33): the public header
    must give every field the offset the reference's declaration gives it.  Both are compiled by gcc:
    the header as shipped, and the reference's field list restated here with opaque pointers."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("gcc not found")
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stddef.h>
#include <stdio.h>
#include "thcl_hip.h"
typedef struct RefStorage { int device; float *data; void *cl; void *wrapper; long size; int refcount; char flag;
                            void *allocator; void *allocatorContext; struct RefStorage *view; } RefStorage;
typedef struct RefTensor { long *size; long *stride; int nDimension; RefStorage *storage; long storageOffset;
                           int refcount; char flag; int device; } RefTensor;
#define CHECK(T, R, f) if (offsetof(T, f) != offsetof(R, f)) { printf("%s.%s at %zu, reference %zu\n", #T, #f, offsetof(T, f), offsetof(R, f)); bad = 1; }
int main(void) {
  int bad = 0;
  CHECK(THClStorage, RefStorage, device) CHECK(THClStorage, RefStorage, data) CHECK(THClStorage, RefStorage, cl)
  CHECK(THClStorage, RefStorage, wrapper) CHECK(THClStorage, RefStorage, size) CHECK(THClStorage, RefStorage, refcount)
  CHECK(THClStorage, RefStorage, flag) CHECK(THClStorage, RefStorage, allocator) CHECK(THClStorage, RefStorage, allocatorContext)
  CHECK(THClStorage, RefStorage, view)
  CHECK(THClTensor, RefTensor, size) CHECK(THClTensor, RefTensor, stride) CHECK(THClTensor, RefTensor, nDimension)
  CHECK(THClTensor, RefTensor, storage) CHECK(THClTensor, RefTensor, storageOffset) CHECK(THClTensor, RefTensor, refcount)
  CHECK(THClTensor, RefTensor, flag) CHECK(THClTensor, RefTensor, device)
  if (sizeof(THClStorage) != sizeof(RefStorage) || sizeof(THClTensor) != sizeof(RefTensor)) { printf("sizes differ\n"); bad = 1; }
  printf("%zu %zu\n", sizeof(THClStorage), sizeof(THClTensor));
  return bad;
}
''')
    exe = tmp_path / "layout"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-I", os.path.join(root, "include"), str(src), "-o", str(exe)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr          # also: the public header is valid C99 on its own
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout
