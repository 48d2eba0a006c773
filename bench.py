#!/usr/bin/env python
"""Benchmark of the hot path on one MI355X.

A *step* is one pass of the pointwise/reduce sequence of the first benchmark
configuration over resident fp32 tensors of 2^28 elements (the size the
bandwidth target is quoted on):

    x:add(y); x:cmul(y); x:map2_on_gpu(y, z, "x = sqrt(1000*x*x + y*10 + z*z)"); x:sum(); x:max()

Algorithmic bytes per element: 12 + 12 + 16 + 4 + 4 = 48.  ``value`` is those
bytes divided by the wall time of a step (inputs already in HBM).  Each kernel
is also timed with HIP events on the library's stream inside the timed region;
the ``roofline`` object describes the kernel that takes the largest share (the
three-operand expression kernel).  ``detail`` carries the other configurations
(strided map/copy, reductions along a dim, the point-tensor chain, addmm) and,
under ``w_`` names, the operators either side of the path (catalogue ops,
scans, level-1/2 contractions, indexed movement), each with its own effective
GB/s or TFLOP/s.  The CPU baseline is the TH-semantics
restatement (oracle/) on the host's cores over a bounded sample.

Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3
EXPR = "x = sqrt(1000*x*x + y*10 + z*z)"


class Timers:
    """HIP-event pairs on the library's stream; read only after the final sync."""

    def __init__(self, cl):
        self.cl = cl
        self.st = cl.state()
        self.lib = self.st.lib
        self.rt = self.lib.THClState_getClv2(self.st.ptr, 0)
        self.items = []

    def timed(self, name, fn):
        t = self.lib.thcl_rt_timer_new(self.rt)
        self.lib.thcl_rt_timer_start(t)
        r = fn()
        self.lib.thcl_rt_timer_stop(t)
        self.items.append((name, t))
        return r

    def collect(self):
        out = {}
        for name, t in self.items:
            out.setdefault(name, []).append(self.lib.thcl_rt_timer_ms(t))
            self.lib.thcl_rt_timer_free(t)
        self.items = []
        return out


def stats(ms_list, bytes_or_flops, unit):
    ms = np.array(ms_list, dtype=np.float64)
    avg, med, mn = float(ms.mean()), float(np.median(ms)), float(ms.min())
    scale = 1e-9 if unit == "GB/s" else 1e-12
    return {"avg_ms": round(avg, 4), "median_ms": round(med, 4), "min_ms": round(mn, 4),
            "achieved": round(bytes_or_flops / (avg * 1e-3) * scale, 1), "unit": unit}


def cpu_baseline(n_sample, seed_base=1, min_seconds=12.0):
    """The same step on the host with the TH-semantics restatement: contiguous
    cadd/cmul/map2 with all OpenMP threads (TH parallelises those), sum and max
    on one thread in element order (TH's are serial).  Steps are repeated on the
    same arrays until about `min_seconds` of CPU work has been timed."""
    import oracle
    L = oracle.lib()
    x, y, z = (oracle.uniform(seed_base + i, n_sample) for i in range(3))
    vx = oracle.View.contiguous(x)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    steps, first = 0, None
    t0 = time.perf_counter()
    while True:
        L.th_pointwise_contig_omp(C.c_int(oracle.OPS["cadd"]), C.c_float(1.0), p(vx.storage), p(vx.storage), p(y), C.c_long(n_sample))
        L.th_pointwise_contig_omp(C.c_int(oracle.OPS["cmul"]), C.c_float(0.0), p(vx.storage), p(vx.storage), p(y), C.c_long(n_sample))
        L.th_pointwise_contig_omp(C.c_int(oracle.OPS["map2_c1"]), C.c_float(0.0), p(vx.storage), p(y), p(z), C.c_long(n_sample))
        s = oracle.sumall(vx)
        m = oracle.maxall(vx)
        steps += 1
        if first is None:
            first = (s, m)
        dt = time.perf_counter() - t0
        if dt >= min_seconds or steps >= 200:
            break
    # second, labelled row: fp32 addmm on the host through PyTorch's CPU BLAS (Torch7's lineal descendant)
    import torch
    k = 2048
    a, b, c = (torch.from_numpy(oracle.normal(20 + i, k * k, 0.0, 1.0 / np.sqrt(k)).reshape(k, k)) for i in range(3))
    torch.addmm(c, a, b, beta=0.5, alpha=1.0)
    g0, reps = time.perf_counter(), 0
    while time.perf_counter() - g0 < 2.0:
        torch.addmm(c, a, b, beta=0.5, alpha=1.0)
        reps += 1
    gemm_tflops = 2.0 * k ** 3 * reps / (time.perf_counter() - g0) * 1e-12
    fmt = lambda v: float(np.float32(v)) if np.isfinite(v) else str(v)
    return {"value": round(48.0 * n_sample * steps / dt * 1e-9, 3), "unit": "GB/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": f"{steps} steps on 2^{int(np.log2(n_sample))} elements per tensor ({dt:.1f} s of CPU work): cadd/cmul/map2 as dense "
                      f"OpenMP loops on {oracle.num_threads()} threads, sum (fp64 accumulator) and max serial in element order "
                      f"(max stops at the first NaN, as TH does); Torch7's own map2 calls a Lua closure per element and is far slower",
            "seconds": round(dt, 3), "steps": steps, "first_step_sum_max": [fmt(first[0]), fmt(first[1])],
            "addmm_cpu": {"value": round(gemm_tflops, 3), "unit": "TFLOP/s", "kind": "torch.addmm on CPU tensors, fp32, 2048^3",
                          "threads": torch.get_num_threads()}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--log2n", type=int, default=28, help="elements per tensor (2^k) of the headline step")
    ap.add_argument("--no-detail", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-log2n", type=int, default=27)
    ap.add_argument("--pmc-workload", action="store_true",
                    help="run each headline kernel twice plus a same-size copy (counter calibration) and exit; "
                         "meant to run under `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --kernel-trace`")
    ap.add_argument("--pmc-gemm", action="store_true",
                    help="run the two addmm configurations a few times and exit; meant to run under "
                         "`rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE --kernel-trace`")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import cltorch_amd as cl
    import oracle
    if args.pmc_workload:
        return pmc_workload(cl, 1 << args.log2n)
    if args.pmc_gemm:
        return pmc_gemm(cl, oracle)
    T = Timers(cl)
    n = 1 << args.log2n
    X, Y, Z = (cl.ClTensor(oracle.uniform(s, n)) for s in (1, 2, 3))

    pt_sum, pt_max = cl.ClTensor(), cl.ClTensor()   # point tensors: results stay on the device, no stall in a step

    def step(tm=None):
        run = tm.timed if tm else (lambda name, fn: fn())
        run("add", lambda: X.add(Y))
        run("cmul", lambda: X.cmul(Y))
        run("map2", lambda: X.map2_on_gpu(Y, Z, EXPR))
        run("sum", lambda: pt_sum.sum(X))
        run("max", lambda: pt_max.max(X))

    for _ in range(args.warmup):
        step()
    cl.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(T)
    cl.synchronize()
    wall = time.perf_counter() - t0
    per_kernel = T.collect()
    ms_per_step = wall / args.steps * 1e3
    bytes_per_elem = {"add": 12, "cmul": 12, "map2": 16, "sum": 4, "max": 4}
    kernels = {k: stats(v, bytes_per_elem[k] * n, "GB/s") for k, v in per_kernel.items()}
    for k in kernels.values():
        k["frac_of_peak"] = round(k["achieved"] / HBM_PEAK_GBS, 4)
    value = 48.0 * n / (ms_per_step * 1e-3) * 1e-9
    dom = kernels["map2"]
    out = {
        "metric": "effective HBM GB/s (% of peak) for apply/reduce; fp32 addmm TFLOP/s",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"config 1 sequence (add, cmul, map2 '{EXPR}', sum, max) on contiguous fp32 1-D tensors of "
                               f"2^{args.log2n} elements, uniform[-1,1) MT19937 seeds 1,2,3; 48 algorithmic bytes/element/step",
                   "elements": n},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": {"bound": "hbm", "kernel": "thcl_expr3_d6642be2_contig_v4 (the map2 expression, 3 operands)",
                     "achieved": dom["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom["achieved"] / HBM_PEAK_GBS, 4),
                     # HBM bytes per launch from rocprofv3 FETCH_SIZE/WRITE_SIZE, calibrated on a copy kernel
                     # (profiles/headline_kernels_2p28_pmc_traffic.txt): 15.999 bytes/element at 2^28 elements
                     "traffic": int(round(15.999 * n)) if args.log2n == 28 else None,
                     "algorithmic_bytes_per_launch": 16 * n, "avg_launch_ms": dom["avg_ms"]},
        "kernels": kernels,
    }

    if not args.no_detail:
        out["detail"] = detail(cl, oracle, T, X, Y, Z, n)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(1 << args.cpu_log2n)
    print(json.dumps(out))


def pmc_gemm(cl, oracle):
    """Launches for a matrix-core counter run: config 5's square product five times (the clock
    settles over the first launches) and its skinny product thirty times."""
    k = 8192
    sd = 1.0 / np.sqrt(k)
    Am, Bm, Cm = (cl.ClTensor(oracle.normal(s, k * k, 0.0, sd)).resize(k, k) for s in (8, 9, 10))
    for _ in range(5):
        Cm.addmm(0.5, 1.0, Am, Bm)
    cl.synchronize()
    del Am, Bm, Cm
    M, N, K = 64, 16384, 4096
    sd = 1.0 / np.sqrt(K)
    At = cl.ClTensor(oracle.normal(11, K * M, 0.0, sd)).resize(K, M)
    Bs = cl.ClTensor(oracle.normal(12, K * N, 0.0, sd)).resize(K, N)
    Cs = cl.ClTensor(oracle.normal(13, M * N, 0.0, sd)).resize(M, N)
    for _ in range(30):
        Cs.addmm(0.5, 1.0, At.t(), Bs)
    cl.synchronize()
    print(json.dumps({"pmc_gemm": "done"}))


def pmc_workload(cl, n):
    """Launches for hardware-counter runs: a copy between the two halves of one
    storage (runs the library's dense copy kernel: reads 4n bytes, writes 4n
    bytes -- the calibration point for FETCH_SIZE / WRITE_SIZE) and the five
    kernels of the headline step, twice."""
    rng = np.random.RandomState(0)
    x = rng.uniform(-1, 1, n).astype(np.float32)
    X, Y, Z = cl.ClTensor(x), cl.ClTensor(x[::-1].copy()), cl.ClTensor(np.abs(x))
    W = cl.ClTensor(2 * n)
    lo, hi = W.narrow(1, 1, n), W.narrow(1, n + 1, n)
    lo.copy(X)
    pt = cl.ClTensor()
    for _ in range(2):
        hi.copy(lo)
        X.add(Y)
        X.cmul(Y)
        X.map2_on_gpu(Y, Z, EXPR)
        pt.sum(X)
        pt.max(X)
    cl.synchronize()
    print(json.dumps({"pmc_workload": "done", "elements": n}))


def detail(cl, oracle, T, X, Y, Z, n):
    """The other benchmark configurations, a few launches each."""
    d = {}
    reps = 20

    def measure(name, fn, work, unit="GB/s", reps=reps, peak=HBM_PEAK_GBS):
        fn()
        cl.synchronize()
        for _ in range(reps):
            T.timed(name, fn)
        cl.synchronize()
        s = stats(T.collect()[name], work, unit)
        s["frac_of_peak"] = round(s["achieved"] / peak, 4)
        d[name] = s

    # config 4: reduce-all into a point tensor, then pointwise ops fed by it, no host sync in between
    pt = cl.ClTensor()
    A = X
    A.copy(cl.ClTensor(oracle.uniform(7, n, 0.0, 1.0)))
    measure("c4_sumall_gpu_2^%d" % int(np.log2(n)), lambda: pt.sum(A), 4 * n)
    measure("c4_div_point_tensor", lambda: A.div(pt) and pt.sum(A), 12 * n)   # div (8 B) + the sum that feeds the next div (4 B)
    chain = [lambda: A.mul(1.0001), lambda: A.add(0.5), lambda: A.cmul(A), lambda: A.sqrt(), lambda: A.add(pt),
             lambda: A.mul(pt), lambda: A.abs(), lambda: A.csub(0.25)]
    cl.synchronize()
    t0 = time.perf_counter()
    T.timed("c4_chain_10_launches", lambda: [pt.sum(A), A.div(pt)] + [f() for f in chain])
    cl.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    ms = T.collect()["c4_chain_10_launches"]
    d["c4_chain_10_launches"] = {"gpu_ms": round(ms[0], 3), "wall_ms": round(wall, 3),
                                 "achieved": round((4 + 8 * 9) * n / (ms[0] * 1e-3) * 1e-9, 1), "unit": "GB/s",
                                 "note": "sumall_gpu + div_gpu + 8 in-place ops, one sync at the end"}
    measure("c1_fill", lambda: A.fill(0.5), 4 * n)

    # config 2: strided views of a 512x512x256 tensor
    m = 512 * 512 * 256
    a = cl.ClTensor(oracle.uniform(4, m)).resize(512, 512, 256)
    b = cl.ClTensor(oracle.uniform(5, m)).resize(512, 512, 256)
    aT, bT = a.transpose(1, 3), b.transpose(1, 3)
    measure("c2_map_transposed_views", lambda: aT.map_on_gpu(bT, "x = 1000*x + y*10"), 12 * m)
    dst = cl.ClTensor(256, 512, 512)
    measure("c2_copy_transposed_to_dense", lambda: dst.copy(aT), 8 * m)
    aS = a.strided((512, 512, 128), (131072, 256, 2))
    bS = b.strided((512, 512, 128), (131072, 256, 2))
    measure("c2_map_stride2_views", lambda: aS.map_on_gpu(bS, "x = 1000*x + y*10"), 12 * (m // 2))
    dS = cl.ClTensor(512, 512, 128)
    measure("c2_copy_stride2_to_dense", lambda: dS.copy(aS), 8 * (m // 2))
    aN, bN = a.narrow(3, 65, 128), b.narrow(3, 65, 128)
    measure("c2_map_narrow_views", lambda: aN.map_on_gpu(bN, "x = 1000*x + y*10"), 12 * (m // 2))
    del a, b, aT, bT, aS, bS, aN, bN, dst, dS

    # config 3: reductions along each dim of 4096 x 16384
    r, c = 4096, 16384
    G = cl.ClTensor(oracle.normal(6, r * c)).resize(r, c)
    for dim, nout in ((1, c), (2, r)):
        measure(f"c3_sum_dim{dim}", lambda: G.sum(dim), 4 * r * c + 4 * nout)
        measure(f"c3_max_dim{dim}", lambda: G.max(dim), 4 * r * c + 8 * nout)
        measure(f"c3_min_dim{dim}", lambda: G.min(dim), 4 * r * c + 8 * nout)
    del G

    # config 5: addmm
    k = 8192
    sd = 1.0 / np.sqrt(k)
    Am, Bm, Cm = (cl.ClTensor(oracle.normal(s, k * k, 0.0, sd)).resize(k, k) for s in (8, 9, 10))
    measure("c5_addmm_8192", lambda: Cm.addmm(0.5, 1.0, Am, Bm), 2.0 * k ** 3, "TFLOP/s", reps=10, peak=FP32_MFMA_PEAK_TFLOPS)
    del Am, Bm, Cm
    M, N, K = 64, 16384, 4096
    At = cl.ClTensor(oracle.normal(11, K * M, 0.0, sd)).resize(K, M)
    Bs = cl.ClTensor(oracle.normal(12, K * N, 0.0, sd)).resize(K, N)
    Cs = cl.ClTensor(oracle.normal(13, M * N, 0.0, sd)).resize(M, N)
    measure("c5_addmm_skinny_64x16384x4096", lambda: Cs.addmm(0.5, 1.0, At.t(), Bs), 2.0 * M * N * K, "TFLOP/s",
            peak=FP32_MFMA_PEAK_TFLOPS)
    d["c5_addmm_skinny_64x16384x4096"]["hbm_GBs"] = round(
        4.0 * (M * K + K * N + 2 * M * N) / (d["c5_addmm_skinny_64x16384x4096"]["avg_ms"] * 1e-3) * 1e-9, 1)
    del At, Bs, Cs

    # the reference's own perf script times 900 calls of cmul / add / sum on 6400- and 64000-element
    # tensors (src/test/test-perf.lua:43-106): per-call cost where launches, not bytes, dominate
    lat = {}
    for m_small in (6400, 64000):
        sa, sb, spt = cl.ClTensor(m_small), cl.ClTensor(m_small), cl.ClTensor()
        sa.fill(1.0)
        sb.fill(1.0)
        for name, fn in (("cmul", lambda: sa.cmul(sb)), ("add", lambda: sa.add(sb)), ("sum_to_point_tensor", lambda: spt.sum(sa)),
                         ("sum_to_host", lambda: sa.sum())):
            fn()
            cl.synchronize()
            t0 = time.perf_counter()
            for _ in range(900):
                fn()
            cl.synchronize()
            lat[f"{name}_{m_small}"] = round((time.perf_counter() - t0) / 900 * 1e6, 2)
    d["small_tensor_us_per_call"] = dict(lat, note="900 calls through the Python mirror, one synchronisation at the end "
                                                   "(sum_to_host waits for every result)")

    # ---- the callers either side of the path: operator catalogue, scans, level-1/2, indexed movement
    A.fill(0.75)
    B = Y
    measure("w_clamp_2^%d" % int(np.log2(n)), lambda: A.clamp(-0.5, 0.5), 8 * n)
    measure("w_lt_tensor", lambda: Z.lt(A, B), 12 * n)
    measure("w_norm2_to_host", lambda: A.norm(2.0), 4 * n)
    measure("w_dot_to_host", lambda: A.dot(B), 8 * n)
    measure("w_cumsum_1d", lambda: Z.cumsum(A, 1), 8 * n)
    G = cl.ClTensor(4096 * 16384).resize(4096, 16384)
    G.fill(0.5)
    R = cl.ClTensor(4096, 16384)
    for dim in (1, 2):
        measure(f"w_cumsum_4096x16384_dim{dim}", lambda: R.cumsum(G, dim), 8 * 4096 * 16384)
    del R
    q = 16384
    Mq = cl.ClTensor(q * q).resize(q, q)
    Mq.fill(0.01)
    v, y = cl.ClTensor(q), cl.ClTensor(q)
    v.fill(1.0)
    y.fill(0.0)
    measure("w_addmv_rowmajor_16384", lambda: y.addmv(0.0, 1.0, Mq, v), 4 * q * q)
    measure("w_addmv_colmajor_16384", lambda: y.addmv(0.0, 1.0, Mq.t(), v), 4 * q * q)
    measure("w_addr_16384", lambda: Mq.addr(1.0, 0.5, v, y), 8 * q * q)
    del Mq
    rows, width, cnt = 100000, 1024, 65536
    rs = np.random.RandomState(0)
    tab = cl.ClTensor(rows * width).resize(rows, width)
    tab.fill(1.0)
    idx = cl.ClTensor(rs.randint(1, rows + 1, size=cnt).astype(np.float32))
    sel = cl.ClTensor(cnt, width)
    measure("w_indexSelect_rows_65536x1024", lambda: sel.index(tab, 1, idx), 8 * cnt * width)
    measure("w_indexCopy_rows_65536x1024", lambda: tab.indexCopy(1, idx, sel), 8 * cnt * width)
    del tab, sel
    # shapes that leave a plain slice-per-block or element-order walk idle: few long slices, a handful of
    # columns, a whole-tensor sum over a transposed view, a ragged product
    few = cl.ClTensor(64 << 20).resize(64, 1 << 20)
    few.fill(0.5)
    res = cl.ClTensor()
    measure("w_sum_dim2_64x2^20", lambda: res.sum(few, 2), 4 * (64 << 20))
    measure("w_max_dim2_64x2^20", lambda: few.max(2), 4 * (64 << 20))
    tall = few.resize(1 << 24, 4)
    measure("w_sum_dim1_2^24x4", lambda: res.sum(tall, 1), 4 * (64 << 20))
    sq = tall.resize(8192, 8192).t()
    measure("w_sumall_transposed_8192^2", lambda: res.sum(sq), 4 * (64 << 20))
    del few, tall, sq
    ra, rb, rc = cl.ClTensor(3000, 7000), cl.ClTensor(7000, 5000), cl.ClTensor(3000, 5000)
    ra.fill(0.01)
    rb.fill(0.02)
    rc.fill(0.0)
    measure("w_addmm_3000x5000x7000", lambda: rc.addmm(0.0, 1.0, ra, rb), 2.0 * 3000 * 5000 * 7000, "TFLOP/s", reps=6,
            peak=FP32_MFMA_PEAK_TFLOPS)
    del ra, rb, rc
    mask = cl.ClTensor((rs.rand(1 << 26) > 0.5).astype(np.float32))
    src = cl.ClTensor(1 << 26)
    src.fill(1.0)
    packed = cl.ClTensor()
    # algorithmic bytes: mask and source read once, half of the source written (the call also
    # waits for the count, which sizes the result)
    measure("w_maskedSelect_2^26_half", lambda: packed.maskedSelect(src, mask), (4 + 4 + 2) * (1 << 26))
    return d


if __name__ == "__main__":
    main()
