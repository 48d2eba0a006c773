"""GPU parity: pointwise apply, expressions and copies against the CPU oracle,
bit for bit, through the C ABI (ctypes mirror of the Lua methods).  Modelled on
the reference's own cases (src/test/unit_tensor.lua:225-359,583-635,759-775)."""
import os

import numpy as np
import pytest

import oracle
from oracle import View, expr_host
from gpu_util import Pair, assert_bit_equal

pytestmark = pytest.mark.gpu
F = np.float32

SIZES = [1, 2, 3, 4, 5, 63, 64, 65, 255, 1023, 1024, 1025, 4096 + 3, 100003, (1 << 20) + 1]


def _ops():
    # name, device call, oracle op, oracle scalar
    return [
        ("add(y)", lambda X, Y: X.add(Y), "cadd", 1.0),
        ("add(0.3,y)", lambda X, Y: X.add(0.3, Y), "cadd", float(F(0.3))),
        ("csub(y)", lambda X, Y: X.csub(Y), "csub", 1.0),
        ("csub(0.7,y)", lambda X, Y: X.csub(0.7, Y), "csub", float(F(0.7))),
        ("cmul(y)", lambda X, Y: X.cmul(Y), "cmul", 0.0),
        ("cdiv(y)", lambda X, Y: X.cdiv(Y), "cdiv", 0.0),
    ]


@pytest.mark.parametrize("n", SIZES)
def test_inplace_binary_dense_all_lengths(cl, n):
    x, y = oracle.uniform(1, n), oracle.uniform(2, n, 0.5, 1.5)
    for name, dev, op, v in _ops():
        px, py = Pair.dense(cl, x), Pair.dense(cl, y)
        dev(px.dev, py.dev)
        oracle.pointwise(op, px.view, px.view, py.view, v)
        assert_bit_equal(px.device_storage(), px.host_storage, f"{name} n={n}")
        assert_bit_equal(py.device_storage(), y, "input modified")


def test_reference_small_matrices(cl, golden):
    c = np.array(golden["pointwise_pairs"]["c"], dtype=F)
    d = np.array(golden["pointwise_pairs"]["d"], dtype=F)
    assert_bit_equal(cl.ClTensor(c).add(cl.ClTensor(d)).float(), c + d)
    assert_bit_equal(cl.ClTensor(c).cmul(cl.ClTensor(d)).float(), c * d)
    assert_bit_equal(cl.ClTensor(c).cdiv(cl.ClTensor(d)).float(), c / d)
    # out-of-place forms resize the result (torch.add(c, d))
    r = cl.ClTensor()
    r.add(cl.ClTensor(c), cl.ClTensor(d))
    assert r.size() == (2, 3)
    assert_bit_equal(r.float(), c + d)
    r = cl.ClTensor()
    r.cmul(cl.ClTensor(c), cl.ClTensor(d))
    assert_bit_equal(r.float(), c * d)
    g = golden["user_kernel_add3"]
    assert cl.ClTensor(g["x"]).apply_on_gpu(g["expr"]).float().tolist() == g["expect"]


def test_scalar_forms(cl, golden):
    c = np.array(golden["scalar_ops"]["c"], dtype=F)
    v = golden["scalar_ops"]["value"]
    fv = F(v)
    assert_bit_equal(cl.ClTensor(c).add(v).float(), c + fv)
    assert_bit_equal(cl.ClTensor(c).csub(v).float(), c + (-fv))
    assert_bit_equal(cl.ClTensor(c).mul(v).float(), c * fv)
    assert_bit_equal(cl.ClTensor(c).div(v).float(), c / fv)        # true division, Torch7's CPU result
    r = cl.ClTensor()
    r.mul(cl.ClTensor(c), v)
    assert_bit_equal(r.float(), c * fv)
    x = oracle.uniform(4, 100001)
    assert_bit_equal(cl.ClTensor(x).div(3.4).float(), x / F(3.4))
    assert_bit_equal(cl.ClTensor(x).fill(1.345).float(), np.full_like(x, F(1.345)))
    assert_bit_equal(cl.ClTensor(x).zero().float(), np.zeros_like(x))


def test_unary_fixed_ops(cl, golden):
    c = np.array(golden["pointwise_unary"]["c"], dtype=F)
    with np.errstate(invalid="ignore"):
        assert_bit_equal(cl.ClTensor(c).sqrt().float(), np.sqrt(c))
    assert_bit_equal(cl.ClTensor(c).abs().float(), np.abs(c))
    assert_bit_equal(cl.ClTensor(c).neg().float(), -c)
    assert_bit_equal(cl.ClTensor(c).cinv().float(), F(1) / c)
    r = cl.ClTensor()
    r.abs(cl.ClTensor(c))
    assert_bit_equal(r.float(), np.abs(c))
    # transcendental operators: the reference's own tolerance (abs 2e-4, src/test/unit_tensor.lua:73-93)
    tol = golden["tolerances"]["float_abs"]
    pos = np.abs(c) + F(0.5)
    assert np.allclose(cl.ClTensor(c).exp().float(), np.exp(c), atol=tol, rtol=1e-6)
    assert np.allclose(cl.ClTensor(pos).log().float(), np.log(pos), atol=tol)
    assert np.allclose(cl.ClTensor(c).tanh().float(), np.tanh(c), atol=tol)
    assert np.allclose(cl.ClTensor(c).sigmoid().float(), 1 / (1 + np.exp(-c)), atol=tol)
    assert_bit_equal(cl.ClTensor(c).floor().float(), np.floor(c))
    assert_bit_equal(cl.ClTensor(c).ceil().float(), np.ceil(c))


def test_three_tensor_forms(cl):
    n = 70001
    a, b, t = oracle.uniform(1, n), oracle.uniform(2, n, 0.5, 1.5), oracle.uniform(3, n)
    A, B = cl.ClTensor(a), cl.ClTensor(b)
    assert_bit_equal(cl.ClTensor().add(A, 0.25, B).float(), a + F(0.25) * b)
    assert_bit_equal(cl.ClTensor().csub(A, B).float(), a - b)
    assert_bit_equal(cl.ClTensor().cdiv(A, B).float(), a / b)
    assert_bit_equal(cl.ClTensor(t).addcmul(0.5, A, B).float(), t + F(0.5) * a * b)
    assert_bit_equal(cl.ClTensor(t).addcdiv(0.5, A, B).float(), t + F(0.5) * a / b)
    r = cl.ClTensor()
    r.addcmul(cl.ClTensor(t), 2.0, A, B)
    assert_bit_equal(r.float(), t + F(2.0) * a * b)


@pytest.mark.parametrize("misalign", [1, 2, 3])
def test_dense_but_misaligned_views(cl, misalign):
    n = 50000
    x, y = oracle.uniform(1, n + 8), oracle.uniform(2, n + 8)
    px = Pair(cl, x, misalign, (n,), (1,))
    py = Pair(cl, y, (misalign * 2) % 4, (n,), (1,))
    px.dev.add(py.dev)
    oracle.pointwise("cadd", px.view, px.view, py.view, 1.0)
    assert_bit_equal(px.device_storage(), px.host_storage, "outside the view must stay untouched")


def _strided_cases(cl):
    """(name, Pair x, Pair y) with equal shapes, covering each kernel family."""
    rng_x = oracle.uniform(4, 24 * 40 * 16)
    rng_y = oracle.uniform(5, 24 * 40 * 16)
    base_x = Pair.dense(cl, rng_x.reshape(24, 40, 16))
    base_y = Pair.dense(cl, rng_y.reshape(24, 40, 16))
    yield "both transposed alike", base_x.transpose(0, 2), base_y.transpose(0, 2)
    yield "x transposed, y dense", base_x.transpose(0, 2), Pair.dense(cl, rng_y.reshape(16, 40, 24))
    yield "x dense, y transposed", Pair.dense(cl, rng_x.reshape(16, 40, 24)), base_y.transpose(0, 2)
    yield "stride 2 inner", base_x.step(2, 2), base_y.step(2, 2)
    yield "narrow inner aligned", base_x.narrow(2, 4, 8), base_y.narrow(2, 8, 8)
    yield "narrow inner misaligned", base_x.narrow(2, 1, 7), base_y.narrow(2, 3, 7)
    yield "narrow middle", base_x.narrow(1, 3, 21), base_y.narrow(1, 5, 21)
    yield "select-like", base_x.narrow(0, 5, 1), base_y.narrow(0, 7, 1)
    yield "transpose(1,2)", base_x.transpose(1, 2), base_y.transpose(1, 2).narrow(0, 0, 24)


def test_strided_binary_ops_joint_layouts(cl):
    for name, px, py in _strided_cases(cl):
        before_y = py.host_storage.copy()
        px.dev.add(py.dev)
        oracle.pointwise("cadd", px.view, px.view, py.view, 1.0)
        assert_bit_equal(px.device_storage(), px.host_storage, name)
        px.dev.map_on_gpu(py.dev, "x = 1000*x + y*10")
        oracle.pointwise("map_c2", px.view, py.view)
        assert_bit_equal(px.device_storage(), px.host_storage, name + " (expression)")
        assert_bit_equal(py.device_storage(), before_y, name + " input")


def test_operands_of_different_shapes_pair_by_position(cl):
    # only the element counts agree (src/lib/THClApply.cpp:152-159)
    x = oracle.uniform(6, 30 * 28)
    y = oracle.uniform(7, 30 * 28 * 2)
    px = Pair.dense(cl, x.reshape(30, 28))
    py = Pair(cl, y, 0, (28, 30), (1, 56))          # transposed, gapped, different shape
    px.dev.add(py.dev)
    oracle.pointwise("cadd", px.view, px.view, py.view, 1.0)
    assert_bit_equal(px.device_storage(), px.host_storage)
    pz = Pair(cl, y, 1, (4, 7, 30), (2, 8, 56))     # last element at 1 + 6 + 48 + 1624 = 1679, inside the storage
    px.dev.map2_on_gpu(py.dev, pz.dev, "x = x*y + z")
    want = expr_host.evaluate("x = x*y + z", px.view.gather().reshape(-1), py.view.gather().reshape(-1),
                              pz.view.gather().reshape(-1))
    assert_bit_equal(px.device_storage(), want)


def test_many_dimensions(cl):
    sizes = (2, 3, 2, 2, 3, 2, 2, 2, 3, 2)
    n = int(np.prod(sizes))
    x, y = oracle.uniform(8, n * 2), oracle.uniform(9, n)
    strides, z = [], 2
    for s in reversed(sizes):
        strides.append(z)
        z *= s
    strides = tuple(reversed(strides))              # every element 2 apart: collapses to one strided dim
    px = Pair(cl, x, 1, sizes, strides)
    py = Pair.dense(cl, y.reshape(sizes))
    px.dev.cmul(py.dev)
    oracle.pointwise("cmul", px.view, px.view, py.view)
    assert_bit_equal(px.device_storage(), px.host_storage)
    # non-collapsible: reverse the dims of a dense tensor
    rev = tuple(range(len(sizes) - 1, -1, -1))
    base = Pair.dense(cl, y.reshape(sizes))
    v = View(base.host_storage, 0, tuple(sizes[i] for i in rev), tuple(base.view.strides[i] for i in rev))
    pr = base.derive(v)
    out = Pair.dense(cl, np.zeros(v.sizes, dtype=F))
    out.dev.copy(pr.dev)
    oracle.pointwise("copy", out.view, pr.view)
    assert_bit_equal(out.device_storage(), out.host_storage)
    with pytest.raises(cl.ClError):
        cl.ClTensor(4).add(cl.ClTensor(5))


def test_written_operand_that_overlaps_itself(cl):
    # expanded (stride 0) destination: staged through a dense temporary, then
    # scattered back; every alias ends up with one of the written values
    x = oracle.uniform(10, 8)
    px = Pair(cl, x, 0, (4, 8), (0, 1))
    y = oracle.uniform(11, 32).reshape(4, 8)
    px.dev.add(cl.ClTensor(y))
    got = px.device_storage()
    candidates = x.reshape(1, 8) + y
    assert all(any(got[j] == candidates[i, j] for i in range(4)) for j in range(8))


def test_point_tensor_operands(cl):
    n = 100003
    a = oracle.uniform(7, n, 0.0, 1.0)
    A = cl.ClTensor(a)
    s = cl.ClTensor()
    s.sum(A)                                   # stays on the device
    assert s.nDimension() == 0
    sv = F(s.s())
    assert_bit_equal(cl.ClTensor(a).div(s).float(), a / sv)
    assert_bit_equal(cl.ClTensor(a).mul(s).float(), a * sv)
    assert_bit_equal(cl.ClTensor(a).add(s).float(), a + sv)     # cadd with a point tensor on the right
    assert_bit_equal(cl.ClTensor(a).csub(s).float(), a - sv)
    assert_bit_equal(cl.ClTensor(n).fill(s).float(), np.full(n, sv, dtype=F))
    r = cl.ClTensor()
    r.div(A, s)
    assert_bit_equal(r.float(), a / sv)


EXPRS = [
    ("x = sqrt(1000*x*x + y*10 + z*z)", 3, True),
    ("*out = sqrt(*out * *out + *in1 * *in1 + *in2 + 3 + exp(*in2))", 3, False),
    ("x = sqrt(x * x + y * y + z + 3 + exp(z))", 3, False),
    ("x = 1000*x + y*10", 2, True),
    ("*out = sqrt(*out * *out + *in1 * *in1 + 3 + exp(*in1))", 2, False),
    ("x = sqrt(x + 3) + exp(x)", 1, False),
    ("x = x * 0.5 + 1e-3", 1, True),
    ("x = (x > 0.25) ? x : 2*x", 1, True),
    ("x = max(x, y) - min(x, y)", 2, True),
]


@pytest.mark.parametrize("expr,nt,exact", EXPRS)
def test_user_expressions(cl, golden, expr, nt, exact):
    n = 60 * 50
    arrs = [oracle.uniform(20 + i, n, -0.5, 0.5) for i in range(3)][:nt]
    T = [cl.ClTensor(a.reshape(60, 50)) for a in arrs]
    if nt == 1:
        T[0].apply_on_gpu(expr)
    elif nt == 2:
        T[0].map_on_gpu(T[1], expr)
    else:
        T[0].map2_on_gpu(T[1], T[2], expr)
    want = expr_host.evaluate(expr, *arrs)
    got = T[0].float().reshape(-1)
    if exact:
        assert_bit_equal(got, want, expr)
    else:
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.max(np.abs(got[ok] - want[ok])) <= golden["tolerances"]["float_abs"], expr


def test_expression_aliases_and_errors(cl):
    x, y = oracle.uniform(1, 1000), oracle.uniform(2, 1000)
    a = cl.ClTensor(x).apply2_on_gpu(cl.ClTensor(y), "x = x - y").float()
    b = cl.ClTensor(x).map_on_gpu(cl.ClTensor(y), "*out = *out - *in1").float()
    assert_bit_equal(a, x - y)
    assert_bit_equal(b, x - y)
    with pytest.raises(cl.ClError, match="compile"):
        cl.ClTensor(x).apply_on_gpu("x = undefined_function_zzz(x)")
    with pytest.raises(cl.ClError):
        cl.ClTensor(x).div(0.0)
    # the library is still usable after an error
    assert_bit_equal(cl.ClTensor(x).add(1.0).float(), x + F(1))


# ------------------------------------------------------------------ copies ---
def test_copies_are_bit_exact_for_every_layout(cl):
    for name, px, _ in _strided_cases(cl):
        dst = Pair.dense(cl, np.zeros(px.view.sizes, dtype=F))
        dst.dev.copy(px.dev)
        assert_bit_equal(dst.device_storage(), px.view.gather(), name + " -> dense")
        back = Pair.dense(cl, np.full(px.view.sizes, F(7)))
        px.dev.copy(back.dev)                   # dense -> strided scatter
        oracle.pointwise("copy", px.view, back.view)
        assert_bit_equal(px.device_storage(), px.host_storage, "dense -> " + name)
    # special values travel unchanged
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38], dtype=F)
    assert np.array_equal(cl.ClTensor(special).clone().float().view(np.uint32), special.view(np.uint32))
    t = Pair.dense(cl, np.tile(special, 8).reshape(8, 8)).transpose(0, 1)
    assert np.array_equal(t.dev.contiguous().float().view(np.uint32),
                          np.tile(special, 8).reshape(8, 8).T.copy().view(np.uint32))


def test_copy_within_one_storage_and_size_checks(cl):
    x = oracle.uniform(3, 64)
    p = Pair(cl, x, 0, (32,), (1,))
    q = p.derive(View(p.host_storage, 32, (32,), (1,)))
    q.dev.copy(p.dev)                           # same storage: goes through the kernel, not a block copy
    assert_bit_equal(p.device_storage(), np.concatenate([x[:32], x[:32]]))
    with pytest.raises(cl.ClError, match="sizes do not match"):
        cl.ClTensor(5).copy(cl.ClTensor(6))
    e = cl.ClTensor()
    e.copy(cl.ClTensor())                       # empty to empty: nothing happens


def test_host_roundtrip_of_strided_views(cl):
    base = oracle.uniform(12, 6 * 8 * 10).reshape(6, 8, 10)
    p = Pair.dense(cl, base)
    assert_bit_equal(p.transpose(0, 2).dev.float(), base.transpose(2, 1, 0))
    assert_bit_equal(p.narrow(1, 2, 3).dev.float(), base[:, 2:5, :])
    t = p.transpose(0, 1)
    t.dev.copy(np.arange(8 * 6 * 10, dtype=F).reshape(8, 6, 10))     # host -> strided device view
    assert_bit_equal(p.dev.float(), np.arange(480, dtype=F).reshape(8, 6, 10).transpose(1, 0, 2))


# ------------------------------------------------- transposed operands (LDS tiles) ---
@pytest.mark.parametrize("shape", [(130, 70), (64, 128), (200, 300), (3, 150, 90), (5, 17, 260), (2, 3, 70, 129),
                                   (64, 300), (300, 64), (256, 1024), (2, 512, 1024), (3, 1024, 272),
                                   (1000, 3000), (4, 128, 132), (100, 60), (2, 3, 68, 260)])
def test_transposed_operand_meets_dense_one(cl, shape):
    """Operands whose unit-stride dims differ: the library stages the transposed
    ones through LDS tiles; full tiles, ragged edges and outer dims, each of the
    three tile shapes (thin dims pick 256 x 64 or 64 x 256) and the diagonal
    tile order that power-of-two pitches switch on."""
    n = int(np.prod(shape))
    nd = len(shape)
    x, y, z = oracle.uniform(31, n), oracle.uniform(32, n), oracle.uniform(33, n)
    tshape = shape[:-2] + (shape[-1], shape[-2])
    # dense destination, source = last two dims transposed
    dst = Pair.dense(cl, np.zeros(shape, dtype=F))
    srcT = Pair.dense(cl, y.reshape(tshape)).transpose(nd - 2, nd - 1)
    dst.dev.copy(srcT.dev)
    assert_bit_equal(dst.device_storage(), srcT.view.gather(), f"copy T->dense {shape}")
    # transposed destination, dense source (scatter through the same kernel)
    dstT = Pair.dense(cl, np.zeros(tshape, dtype=F)).transpose(nd - 2, nd - 1)
    src = Pair.dense(cl, x.reshape(shape))
    dstT.dev.copy(src.dev)
    oracle.pointwise("copy", dstT.view, src.view)
    assert_bit_equal(dstT.device_storage(), dstT.host_storage, f"copy dense->T {shape}")
    # read-write destination
    acc = Pair.dense(cl, x.reshape(shape))
    acc.dev.add(0.5, srcT.dev)
    oracle.pointwise("cadd", acc.view, acc.view, srcT.view, 0.5)
    assert_bit_equal(acc.device_storage(), acc.host_storage, f"cadd {shape}")
    # three operands: one transposed input, one dense; then both transposed
    z_d = Pair.dense(cl, z.reshape(shape))
    acc.dev.map2_on_gpu(srcT.dev, z_d.dev, "x = x*y + z")
    want = expr_host.evaluate("x = x*y + z", acc.view.gather(), srcT.view.gather(), z_d.view.gather())
    assert_bit_equal(acc.device_storage(), want, f"map2 T,dense {shape}")
    zT = Pair.dense(cl, z.reshape(tshape)).transpose(nd - 2, nd - 1)
    acc2 = Pair.dense(cl, x.reshape(shape))
    acc2.dev.addcmul(2.0, srcT.dev, zT.dev)
    oracle.pointwise("addcmul", acc2.view, srcT.view, zT.view, 2.0)
    assert_bit_equal(acc2.device_storage(), acc2.host_storage, f"addcmul T,T {shape}")
    assert_bit_equal(srcT.device_storage(), y, "input modified")


def test_transposed_operand_alignment_and_repeats(cl):
    """The 128-bit form of the tiled kernels needs aligned bases and strides; views that
    start an odd number of elements in, rows an odd pitch apart, and operands repeated
    along an outer dim or along the destination's unit-stride dim all give the same
    results through whichever form takes them."""
    rng = np.random.RandomState(77)
    buf_y = rng.standard_normal(4 + 136 * 260).astype(F)
    buf_z = rng.standard_normal(4 + 132 * 264).astype(F)
    for off_y, pitch_y, off_z in ((0, 136, 0), (1, 136, 0), (0, 133, 0), (4, 136, 3), (0, 136, 4)):
        # destination 128 x 256 dense; y = transposed view of a 256 x pitch buffer; z dense rows of pitch 264
        dst = Pair.dense(cl, rng.standard_normal((128, 256)).astype(F))
        py = Pair(cl, buf_y, off_y, (128, 256), (1, pitch_y))
        pz = Pair(cl, buf_z, off_z, (128, 256), (264, 1))
        dst.dev.map2_on_gpu(py.dev, pz.dev, "x = x + 2*y - z")
        want = expr_host.evaluate("x = x + 2*y - z", dst.view.gather(), py.view.gather(), pz.view.gather())
        assert_bit_equal(dst.device_storage(), want, f"offsets {off_y},{off_z} pitch {pitch_y}")
    # y repeated along the outer dim (stride 0), z repeated along the destination's unit-stride dim
    dst = Pair.dense(cl, rng.standard_normal((3, 64, 128)).astype(F))
    py = Pair(cl, buf_y, 0, (3, 64, 128), (0, 1, 136))
    pz = Pair(cl, buf_z, 0, (3, 64, 128), (64, 1, 0))
    dst.dev.map2_on_gpu(py.dev, pz.dev, "x = x*y + z")
    want = expr_host.evaluate("x = x*y + z", dst.view.gather(), py.view.gather(), pz.view.gather())
    assert_bit_equal(dst.device_storage(), want, "repeated operands")
    dst2 = Pair.dense(cl, np.zeros((3, 64, 128), dtype=F))
    dst2.dev.copy(py.dev)
    assert_bit_equal(dst2.device_storage(), py.view.gather(), "copy of a repeated transposed operand")


def test_same_expression_on_every_kernel_family(cl):
    """One expression string, five layouts: the run-time kernel cache must hand
    back the kernel that matches each layout."""
    expr = "x = x*0.5 + y"
    base = oracle.uniform(41, 96 * 80)
    other = oracle.uniform(42, 96 * 80 * 2)

    def run(px, py):
        px.dev.map_on_gpu(py.dev, expr)
        want = expr_host.evaluate(expr, px.view.gather(), py.view.gather())
        oracle.pointwise("copy", px.view, View.contiguous(want))
        assert_bit_equal(px.device_storage(), px.host_storage)

    for _ in range(2):
        run(Pair.dense(cl, base.reshape(96, 80)), Pair.dense(cl, other[:7680].reshape(96, 80)))            # dense 128-bit
        run(Pair(cl, base, 1, (7000,), (1,)), Pair(cl, other, 2, (7000,), (1,)))                            # dense, misaligned
        run(Pair.dense(cl, base.reshape(96, 80)).narrow(1, 8, 32), Pair.dense(cl, other[:7680].reshape(96, 80)).narrow(1, 4, 32))  # joint 128-bit
        run(Pair.dense(cl, base.reshape(96, 80)).step(1, 2), Pair.dense(cl, other[:7680].reshape(96, 80)).step(1, 2))              # joint scalar
        run(Pair.dense(cl, base.reshape(96, 80)), Pair.dense(cl, other[:7680].reshape(80, 96)).transpose(0, 1))                    # tiled
        run(Pair.dense(cl, base.reshape(96, 80)), Pair(cl, other, 0, (80, 96), (1, 160)))                   # different shapes: generic


def test_reshape_copies_in_logical_order(cl):
    x = oracle.uniform(120, 6 * 8 * 5).reshape(6, 8, 5)
    p = Pair.dense(cl, x).transpose(0, 2)                       # 5 x 8 x 6 view
    r = p.dev.reshape(40, 6)
    assert r.size() == (40, 6) and r.isContiguous()
    assert_bit_equal(r.float(), p.view.gather().reshape(40, 6), "reshape of a transposed view")
    with pytest.raises(cl.ClError):
        p.dev.reshape(7, 7)



def test_compiled_kernels_persist_in_the_optional_disk_cache(cl, tmp_path):
    """THCL_KERNEL_CACHE_DIR: the first process compiles and stores the code object, the
    second loads it (same results, file untouched)."""
    import subprocess
    import sys
    code = ("import numpy as np, cltorch_amd as cl\n"
            "x = cl.ClTensor(np.arange(8, dtype=np.float32))\n"
            "x.apply_on_gpu('x = x*3 + 0.125')\n"
            "print(x.float().tolist())\n")
    env = dict(os.environ, THCL_KERNEL_CACHE_DIR=str(tmp_path), PYTHONPATH=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    want = str([float(v * 3 + 0.125) for v in range(8)])
    first = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert first.returncode == 0 and want in first.stdout, first.stderr[-500:]
    files = sorted(tmp_path.glob("thcl_*.hsaco"))
    assert len(files) == 1 and files[0].stat().st_size > 1000
    stamp = files[0].stat().st_mtime_ns
    second = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert second.returncode == 0 and want in second.stdout, second.stderr[-500:]
    assert sorted(tmp_path.glob("thcl_*")) == files and files[0].stat().st_mtime_ns == stamp
    # a damaged file is recompiled over, not trusted
    files[0].write_bytes(b"not a code object")
    third = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert third.returncode == 0 and want in third.stdout, third.stderr[-500:]
    assert files[0].stat().st_size > 1000


def test_denormal_operands_and_results_are_kept(cl):
    """Subnormal fp32 values are neither flushed on input nor on output, in fixed
    operators and in run-time compiled expressions alike."""
    x = np.array([1e-39, 3e-42, 1.1754944e-38, -2e-40, 1e-20, 5e-45, 0.0, -0.0], dtype=F)
    y = np.array([0.5, 3.0, 0.5, 2.0, 1e-20, 0.5, 1e-45, -1.0], dtype=F)
    X, Y = cl.ClTensor(x), cl.ClTensor(y)
    with np.errstate(all="ignore"):
        assert_bit_equal(X.clone().cmul(Y).float(), x * y, "cmul")
        assert_bit_equal(X.clone().add(Y).float(), x + y, "add")
        assert_bit_equal(X.clone().cdiv(Y).float(), x / y, "cdiv")
        assert_bit_equal(X.clone().abs().sqrt().float(), np.sqrt(np.abs(x)), "sqrt")
        assert_bit_equal(X.clone().mul(0.25).float(), x * F(0.25), "mul scalar")
        want = expr_host.evaluate("x = x*y + x", x.copy(), y)
        assert_bit_equal(X.clone().map_on_gpu(Y, "x = x*y + x").float(), want, "expression")
    assert X.sum() == float(np.float32(x.astype(np.float64).sum()))
    assert X.min() == float(x.min()) and X.max() == float(x.max())
