#!/usr/bin/env python
"""Benchmark of the hot path on one MI355X.

A *step* is one pass of the pointwise/reduce sequence of the first benchmark
configuration over resident fp32 tensors of 2^28 elements (the size the
bandwidth target is quoted on):

    x:add(y); x:cmul(y); x:map2_on_gpu(y, z, "x = sqrt(1000*x*x + y*10 + z*z)"); x:sum(); x:max()

Algorithmic bytes per element: 12 + 12 + 16 + 4 + 4 = 48.  ``value`` is those
bytes divided by the wall time of a step (inputs already in HBM).  The kernel
that takes the largest share (the three-operand expression kernel) is timed with
a HIP-event pair on the library's stream inside the timed steps and described by
the ``roofline`` object; the other four kernels get their event pairs in a second
pass of the same steps after the timed region, because five pairs cost a step
35-40 us (``ms_per_step_all_pairs`` is that pass).  ``detail`` carries the other configurations
(strided map/copy, reductions along a dim, the point-tensor chain, addmm) and,
under ``w_`` names, the operators either side of the path (catalogue ops,
scans, level-1/2 contractions, indexed movement), each with its own effective
GB/s or TFLOP/s (timed back to back, see ``detail``).  The CPU baseline is the
TH-semantics restatement (oracle/) on the host's cores over a bounded sample;
that leg also runs one step of the same sample on the GPU and compares sum and
max with the NaNs set to zero.  ``roofline.traffic`` and the ``kernel_only_ms``
fields are read from the committed summary of the counter runs
(``profiles/``), which this script also produces:

    rocprofv3 --kernel-trace --stats ... -- python3 bench.py --pmc-configs      (and --pmc FETCH_SIZE / WRITE_SIZE)
    python3 bench.py --summarise TRACE_DB FETCH_DB WRITE_DB > profiles/...txt
    python3 bench.py --pmc-gemm / --summarise-mfma, --summarise-trace

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
    steps, first, first_clean = 0, None, None
    x0 = x.copy()
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
            t_pause = time.perf_counter()
            # the configuration's own sqrt of negative arguments leaves NaNs, so sum and max of a step are NaN on
            # both sides; the same two reductions with the NaNs set to zero give numbers that can be compared
            clean = np.where(np.isnan(vx.storage), np.float32(0), vx.storage)
            vc = oracle.View.contiguous(clean)
            first_clean = (oracle.sumall(vc), oracle.maxall(vc), int(np.isnan(vx.storage).sum()))
            del clean, vc
            t0 += time.perf_counter() - t_pause          # not part of the timed work
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
            "first_step_nan_free": {"sum": float(np.float32(first_clean[0])), "max": float(first_clean[1]), "nans": first_clean[2]},
            "_inputs": (x0, y, z),
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
    ap.add_argument("--pmc-configs", action="store_true",
                    help="run every configuration's operations 1 + 3 times each behind marker launches and exit; meant to run "
                         "under `rocprofv3 --kernel-trace [--pmc FETCH_SIZE | --pmc WRITE_SIZE]`; writes --manifest")
    ap.add_argument("--manifest", default="pmc_configs_manifest.json",
                    help="where --pmc-configs writes (and --summarise reads) the list of operations")
    ap.add_argument("--summarise", nargs=3, metavar=("TRACE_DB", "FETCH_DB", "WRITE_DB"),
                    help="print the text summary of three rocprofv3 runs of --pmc-configs (no GPU needed)")
    ap.add_argument("--write-path", metavar="WPATH_DB", help="with --summarise: a fourth counter run of --pmc-configs (write requests "
                    "of the L2 to memory, their stall cycles, write latency seen by the vector caches); adds two columns")
    ap.add_argument("--summarise-trace", metavar="TRACE_DB", help="print per-kernel totals of a --kernel-trace --stats run of this script")
    ap.add_argument("--summarise-mfma", metavar="PMC_DB", help="print the matrix-core duty summary of a --pmc-gemm counter run")
    ap.add_argument("--pmc-gemm", action="store_true",
                    help="run the two addmm configurations a few times and exit; meant to run under "
                         "`rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE --kernel-trace`")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.summarise:
        w = "python3 $R/bench.py --pmc-configs --manifest $OUT/pmc_configs_manifest.json"
        cmds = [f"rocprofv3 --kernel-trace --stats -d $OUT/cfg_trace -o t -- {w}",
                f"rocprofv3 --pmc FETCH_SIZE --kernel-trace -d $OUT/cfg_fetch -o f -- {w}",
                f"rocprofv3 --pmc WRITE_SIZE --kernel-trace -d $OUT/cfg_write -o w -- {w}",
                "rocprofv3 --pmc " + " ".join(WPATH_COUNTERS) + f" --kernel-trace -d $OUT/cfg_wpath -o p -- {w}",
                "python3 bench.py --manifest $OUT/pmc_configs_manifest.json --summarise $OUT/cfg_trace/t_results.db "
                "$OUT/cfg_fetch/f_results.db $OUT/cfg_write/w_results.db --write-path $OUT/cfg_wpath/p_results.db > " + PROFILE_SUMMARY]
        sys.stdout.write(summarise(*args.summarise, args.manifest, cmds, args.write_path))
        return
    if args.summarise_trace:
        sys.stdout.write(summarise_trace(args.summarise_trace))
        return
    if args.summarise_mfma:
        sys.stdout.write(summarise_mfma(args.summarise_mfma))
        return
    import cltorch_amd as cl
    import oracle
    if args.pmc_configs:
        return pmc_configs(cl, oracle, 1 << args.log2n, args.manifest)
    if args.pmc_gemm:
        return pmc_gemm(cl, oracle)
    T = Timers(cl)
    n = 1 << args.log2n
    X, Y, Z = (cl.ClTensor(oracle.uniform(s, n)) for s in (1, 2, 3))

    pt_sum, pt_max = cl.ClTensor(), cl.ClTensor()   # point tensors: results stay on the device, no stall in a step

    def step(tm=None, only=None):
        # an event pair costs a launch 3-4 us (five pairs: 35-40 us of a 1.9 ms step), so the timed steps carry one
        # pair, around the dominant kernel; the other four are timed in a pass of their own after the timed region
        run = (lambda name, fn: tm.timed(name, fn) if (only is None or name == only) else fn()) if tm else (lambda name, fn: fn())
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
        step(T, only="map2")
    cl.synchronize()
    wall = time.perf_counter() - t0
    per_kernel = T.collect()
    ms_per_step = wall / args.steps * 1e3
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(T)
    cl.synchronize()
    ms_per_step_all_pairs = (time.perf_counter() - t0) / args.steps * 1e3
    per_kernel = dict(T.collect(), map2=per_kernel["map2"])   # map2: from the timed steps
    bytes_per_elem = {"add": 12, "cmul": 12, "map2": 16, "sum": 4, "max": 4}
    kernels = {k: stats(v, bytes_per_elem[k] * n, "GB/s") for k, v in per_kernel.items()}
    for k in kernels.values():
        k["frac_of_peak"] = round(k["achieved"] / HBM_PEAK_GBS, 4)
    value = 48.0 * n / (ms_per_step * 1e-3) * 1e-9
    dom = kernels["map2"]
    prof = committed_profile()
    map2_prof = prof.get("ops", {}).get("c1_map2") if prof.get("elements") == n else None
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
                     # HBM bytes per launch: rocprofv3 FETCH_SIZE + WRITE_SIZE scaled on a dense copy of known size, read
                     # from the committed summary of the counter runs (null when that summary covers another size)
                     "traffic": (map2_prof["read_bytes"] + map2_prof["written_bytes"]) if map2_prof else None,
                     "traffic_source": (PROFILE_SUMMARY + " (operation c1_map2)") if map2_prof else None,
                     "algorithmic_bytes_per_launch": 16 * n, "avg_launch_ms": dom["avg_ms"]},
        "kernels": kernels,
        "kernels_note": "map2 is timed by an event pair inside the timed steps; add, cmul, sum and max in a second pass of "
                        "the same steps with a pair around every kernel (ms_per_step_all_pairs)",
        "ms_per_step_all_pairs": round(ms_per_step_all_pairs, 4),
    }

    if not args.no_detail:
        d = detail(cl, oracle, T, X, Y, Z, n)
        # the rows of the five benchmark configurations go last, so that they sit in the tail of the line
        out["detail"] = dict([(k, v) for k, v in d.items() if not k.startswith("c")] + [(k, v) for k, v in d.items() if k.startswith("c")])
        out["roofline"]["configs"] = config_summary(kernels, d, prof if prof.get("elements") == n else {})
        out["roofline"]["configs_note"] = ("per operation of the five configurations: frac = algorithmic bytes (or flops) / time / peak with "
                                           "calls in a row timed live (ms); kernel_us and traffic (HBM bytes moved / algorithmic bytes) from "
                                           "the committed rocprofv3 summary " + PROFILE_SUMMARY + ", whose own frac is work / kernel_us / peak")
        out["roofline"] = out.pop("roofline")          # after `detail` in the line
    if not args.no_cpu:
        del X, Y, Z
        base = cpu_baseline(1 << args.cpu_log2n)
        # the GPU on the baseline's own sample: one step, NaNs set to zero on the device, same two reductions
        x0, y0, z0 = base.pop("_inputs")
        Xs, Ys, Zs = cl.ClTensor(x0), cl.ClTensor(y0), cl.ClTensor(z0)
        Xs.add(Ys).cmul(Ys).map2_on_gpu(Ys, Zs, EXPR)
        nans = Xs.ne(Xs).sum()                      # a count returned as fp32: exact up to 2^24, rounded once beyond
        Xs.apply_on_gpu("x = (x != x) ? 0.0 : x")
        gs, gm = Xs.sum(), Xs.max()
        want = base["first_step_nan_free"]
        base["gpu_on_same_sample"] = {"sum": gs, "max": gm, "nans": nans,
                                      "sum_rel_diff": abs(gs - want["sum"]) / max(abs(want["sum"]), 1e-30),
                                      "max_equal": gm == want["max"], "nans_equal": nans == float(np.float32(want["nans"]))}
        out["cpu_baseline"] = base
    print(json.dumps(out))


def config_summary(kernels, d, prof):
    """{operation: {frac, ms, kernel_us, traffic}} for every row of the five configurations, a few hundred bytes."""
    ops = prof.get("ops", {})
    out = {}

    def row(name, frac, ms):
        p = ops.get(name)
        r = {"frac": round(frac, 3), "ms": round(ms, 4)}
        if p:
            r["kernel_us"] = round(p["kernel_us"], 1)
            if p["unit"] == "GB/s":
                r["traffic"] = round((p["read_bytes"] + p["written_bytes"]) / p["work"], 3)
        out[name] = r

    for k, v in kernels.items():          # config 1 at the headline size, from the timed steps
        row("c1_" + k, v["frac_of_peak"], v["avg_ms"])
    for name, v in d.items():
        if name.startswith("c") and isinstance(v, dict) and "frac_of_peak" in v:
            row(name, v["frac_of_peak"], v["avg_ms"])
    ch = d.get("c4_chain_10_launches")
    if ch:
        out["c4_chain_10_launches"] = {"frac": round(ch["achieved"] / HBM_PEAK_GBS, 3), "ms": ch["gpu_ms"]}
    return out


def pmc_gemm(cl, oracle):
    """Launches for a matrix-core counter run: config 5's square product five times (the clock
    settles over the first launches), its skinny product 600 times (its time keeps changing over the first
    tens of ms of such work) and two ragged products 12 times each."""
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
    for _ in range(600):
        Cs.addmm(0.5, 1.0, At.t(), Bs)
    cl.synchronize()
    del At, Bs, Cs
    # two ragged products: nothing aligned (4095^3, the kernel with moved-back 16-byte windows) and whole 16-byte
    # groups with edge tiles (3000 x 5000 x 7000); 12 launches each, the summary lists the last
    rs = np.random.RandomState(0)
    for (m_, n_, k_) in ((4095, 4095, 4095), (3000, 5000, 7000)):
        a, b, c = (cl.ClTensor((rs.standard_normal(sh) / np.sqrt(k_)).astype(np.float32)) for sh in ((m_, k_), (k_, n_), (m_, n_)))
        for _ in range(12):
            c.addmm(0.0, 1.0, a, b)
        cl.synchronize()
        del a, b, c
    print(json.dumps({"pmc_gemm": "done"}))


def config_ops(cl, oracle, X, Y, Z, n):
    """The operations of the other configurations and of the callers either side of the path, as a
    generator of (name, fn, work, unit, reps, peak).  Tensors of a group are created when the
    generator reaches it and released when it moves on; ``work`` is algorithmic bytes or flops."""
    H, M = HBM_PEAK_GBS, FP32_MFMA_PEAK_TFLOPS
    lg = int(np.log2(n))
    # config 4: reduce-all into a point tensor, then pointwise ops fed by it, no host sync in between
    pt = cl.ClTensor()
    A = X
    A.copy(cl.ClTensor(oracle.uniform(7, n, 0.0, 1.0)))
    yield ("c4_sumall_gpu_2^%d" % lg, lambda: pt.sum(A), 4 * n, "GB/s", 20, H)
    yield ("c4_div_point_tensor", lambda: A.div(pt) and pt.sum(A), 12 * n, "GB/s", 20, H)   # div (8 B) + the sum that feeds the next div (4 B)
    yield ("c1_fill", lambda: A.fill(0.5), 4 * n, "GB/s", 20, H)

    # config 2: strided views of a 512x512x256 tensor
    m = 512 * 512 * 256
    a = cl.ClTensor(oracle.uniform(4, m)).resize(512, 512, 256)
    b = cl.ClTensor(oracle.uniform(5, m)).resize(512, 512, 256)
    aT, bT = a.transpose(1, 3), b.transpose(1, 3)
    yield ("c2_map_transposed_views", lambda: aT.map_on_gpu(bT, "x = 1000*x + y*10"), 12 * m, "GB/s", 20, H)
    dst = cl.ClTensor(256, 512, 512)
    yield ("c2_copy_transposed_to_dense", lambda: dst.copy(aT), 8 * m, "GB/s", 20, H)
    aS = a.strided((512, 512, 128), (131072, 256, 2))
    bS = b.strided((512, 512, 128), (131072, 256, 2))
    yield ("c2_map_stride2_views", lambda: aS.map_on_gpu(bS, "x = 1000*x + y*10"), 12 * (m // 2), "GB/s", 20, H)
    dS = cl.ClTensor(512, 512, 128)
    yield ("c2_copy_stride2_to_dense", lambda: dS.copy(aS), 8 * (m // 2), "GB/s", 20, H)
    aN, bN = a.narrow(3, 65, 128), b.narrow(3, 65, 128)
    yield ("c2_map_narrow_views", lambda: aN.map_on_gpu(bN, "x = 1000*x + y*10"), 12 * (m // 2), "GB/s", 20, H)
    del a, b, aT, bT, aS, bS, aN, bN, dst, dS

    # config 3: reductions along each dim of 4096 x 16384; the Lua-style call returns new tensors, the
    # `res:sum(src, dim)` form writes into tensors that exist
    r, c = 4096, 16384
    G = cl.ClTensor(oracle.normal(6, r * c)).resize(r, c)
    rv, ri = cl.ClTensor(), cl.ClTensor()
    for dim, nout in ((1, c), (2, r)):
        yield (f"c3_sum_dim{dim}", lambda: G.sum(dim), 4 * r * c + 4 * nout, "GB/s", 20, H)
        yield (f"c3_max_dim{dim}", lambda: G.max(dim), 4 * r * c + 8 * nout, "GB/s", 20, H)
        yield (f"c3_min_dim{dim}", lambda: G.min(dim), 4 * r * c + 8 * nout, "GB/s", 20, H)
        yield (f"c3_sum_dim{dim}_into_existing", lambda: rv.sum(G, dim), 4 * r * c + 4 * nout, "GB/s", 20, H)
        yield (f"c3_max_dim{dim}_into_existing", lambda: rv.max(ri, G, dim), 4 * r * c + 8 * nout, "GB/s", 20, H)
    del G, rv, ri

    # config 5: addmm
    k = 8192
    sd = 1.0 / np.sqrt(k)
    Am, Bm, Cm = (cl.ClTensor(oracle.normal(s, k * k, 0.0, sd)).resize(k, k) for s in (8, 9, 10))
    yield ("c5_addmm_8192", lambda: Cm.addmm(0.5, 1.0, Am, Bm), 2.0 * k ** 3, "TFLOP/s", 10, M)
    del Am, Bm, Cm
    Ms, Ns, Ks = 64, 16384, 4096
    At = cl.ClTensor(oracle.normal(11, Ks * Ms, 0.0, sd)).resize(Ks, Ms)
    Bs = cl.ClTensor(oracle.normal(12, Ks * Ns, 0.0, sd)).resize(Ks, Ns)
    Cs = cl.ClTensor(oracle.normal(13, Ms * Ns, 0.0, sd)).resize(Ms, Ns)
    yield ("c5_addmm_skinny_64x16384x4096", lambda: Cs.addmm(0.5, 1.0, At.t(), Bs), 2.0 * Ms * Ns * Ks, "TFLOP/s", 100, M)
    del At, Bs, Cs

    # ---- the callers either side of the path: operator catalogue, scans, level-1/2, indexed movement
    A.fill(0.75)
    B = Y
    yield ("w_clamp_2^%d" % lg, lambda: A.clamp(-0.5, 0.5), 8 * n, "GB/s", 20, H)
    yield ("w_lt_tensor", lambda: Z.lt(A, B), 12 * n, "GB/s", 20, H)
    yield ("w_norm2_to_host", lambda: A.norm(2.0), 4 * n, "GB/s", 20, H)
    yield ("w_dot_to_host", lambda: A.dot(B), 8 * n, "GB/s", 20, H)
    yield ("w_cumsum_1d", lambda: Z.cumsum(A, 1), 8 * n, "GB/s", 20, H)
    G = cl.ClTensor(4096 * 16384).resize(4096, 16384)
    G.fill(0.5)
    R = cl.ClTensor(4096, 16384)
    for dim in (1, 2):
        yield (f"w_cumsum_4096x16384_dim{dim}", lambda: R.cumsum(G, dim), 8 * 4096 * 16384, "GB/s", 20, H)
    del R, G
    q = 16384
    Mq = cl.ClTensor(q * q).resize(q, q)
    Mq.fill(0.01)
    v, y = cl.ClTensor(q), cl.ClTensor(q)
    v.fill(1.0)
    y.fill(0.0)
    yield ("w_addmv_rowmajor_16384", lambda: y.addmv(0.0, 1.0, Mq, v), 4 * q * q, "GB/s", 20, H)
    yield ("w_addmv_colmajor_16384", lambda: y.addmv(0.0, 1.0, Mq.t(), v), 4 * q * q, "GB/s", 20, H)
    yield ("w_addr_16384", lambda: Mq.addr(1.0, 0.5, v, y), 8 * q * q, "GB/s", 20, H)
    del Mq
    rows, width, cnt = 100000, 1024, 65536
    rs = np.random.RandomState(0)
    tab = cl.ClTensor(rows * width).resize(rows, width)
    tab.fill(1.0)
    idx = cl.ClTensor(rs.randint(1, rows + 1, size=cnt).astype(np.float32))
    sel = cl.ClTensor(cnt, width)
    yield ("w_indexSelect_rows_65536x1024", lambda: sel.index(tab, 1, idx), 8 * cnt * width, "GB/s", 20, H)
    yield ("w_indexCopy_rows_65536x1024", lambda: tab.indexCopy(1, idx, sel), 8 * cnt * width, "GB/s", 20, H)
    del tab, sel
    # shapes that leave a plain slice-per-block or element-order walk idle: few long slices, a handful of
    # columns, a whole-tensor sum over a transposed view, a ragged product
    few = cl.ClTensor(64 << 20).resize(64, 1 << 20)
    few.fill(0.5)
    res = cl.ClTensor()
    yield ("w_sum_dim2_64x2^20", lambda: res.sum(few, 2), 4 * (64 << 20), "GB/s", 20, H)
    yield ("w_max_dim2_64x2^20", lambda: few.max(2), 4 * (64 << 20), "GB/s", 20, H)
    tall = few.resize(1 << 24, 4)
    yield ("w_sum_dim1_2^24x4", lambda: res.sum(tall, 1), 4 * (64 << 20), "GB/s", 20, H)
    sq = tall.resize(8192, 8192).t()
    yield ("w_sumall_transposed_8192^2", lambda: res.sum(sq), 4 * (64 << 20), "GB/s", 20, H)
    del few, tall, sq
    # matrix products outside the configuration: random normal operands like config 5 (constant operands run faster)
    def normal(r, c, k):
        return cl.ClTensor((rs.standard_normal((r, c)) / np.sqrt(k)).astype(np.float32))
    ra, rb, rc = normal(3000, 7000, 7000), normal(7000, 5000, 1), normal(3000, 5000, 1)
    yield ("w_addmm_3000x5000x7000", lambda: rc.addmm(0.0, 1.0, ra, rb), 2.0 * 3000 * 5000 * 7000, "TFLOP/s", 6, M)
    del ra, rb, rc
    # sizes that are no multiple of 4 (16-byte loads without alignment), and a result of 32 rows (128x32 tiles)
    ra, rb, rc = normal(4095, 4095, 4095), normal(4095, 4095, 1), normal(4095, 4095, 1)
    yield ("w_addmm_4095^3", lambda: rc.addmm(0.0, 1.0, ra, rb), 2.0 * 4095 ** 3, "TFLOP/s", 8, M)
    del ra, rb, rc
    ra, rb, rc = normal(32, 4096, 4096), normal(4096, 16384, 1), normal(32, 16384, 1)
    yield ("w_addmm_32x16384x4096", lambda: rc.addmm(0.0, 1.0, ra, rb), 2.0 * 32 * 16384 * 4096, "TFLOP/s", 50, M)
    del ra, rb, rc
    # cubes between the two config-5 shapes: the block tile is picked per shape (whole rounds of tiles per CU)
    for side in (3072, 4608):
        qa, qb, qc = (cl.ClTensor((rs.standard_normal((side, side)) / np.sqrt(side)).astype(np.float32)) for _ in range(3))
        yield ("w_addmm_%d^3" % side, lambda: qc.addmm(0.0, 1.0, qa, qb), 2.0 * side ** 3, "TFLOP/s", 10, M)
        del qa, qb, qc
    mask = cl.ClTensor((rs.rand(1 << 26) > 0.5).astype(np.float32))
    src = cl.ClTensor(1 << 26)
    src.fill(1.0)
    packed = cl.ClTensor()
    # algorithmic bytes: mask and source read once, half of the source written (the call also
    # waits for the count, which sizes the result)
    yield ("w_maskedSelect_2^26_half", lambda: packed.maskedSelect(src, mask), (4 + 4 + 2) * (1 << 26), "GB/s", 20, H)


def detail(cl, oracle, T, X, Y, Z, n):
    """The other benchmark configurations, a few launches each.  Per operation: ``avg_ms`` is one HIP-event pair
    around ``reps`` calls in a row divided by their number -- what a caller that just keeps calling sees, launch
    gaps and result allocation included -- and ``achieved`` / ``frac_of_peak`` follow from it.  ``event_pair_*``
    come from one event pair per call (the pairs' own packets then sit between the calls, which costs a short
    kernel 2-3 us); ``kernel_only_ms`` is the sum of the call's kernel durations in the committed rocprofv3 trace.
    Matrix products get about 40 ms of untimed calls (at least ``reps``) directly in front of the timed ones: the
    clocks settle over the first tens of ms of such work."""
    d = {}
    profiled = committed_profile()
    for name, fn, work, unit, reps, peak in config_ops(cl, oracle, X, Y, Z, n):
        scale = 1e-9 if unit == "GB/s" else 1e-12
        fn()
        cl.synchronize()
        for _ in range(reps):
            T.timed(name, fn)
        cl.synchronize()
        pairs = np.array(T.collect()[name], dtype=np.float64)
        if unit == "TFLOP/s":
            # matrix products: clocks take some tens of ms of such work to settle after a wait or after work of another
            # kind (64x16384x4096 in a row: 96, 112, 94 us per call over the first 30 ms, 85 us from then on)
            for _ in range(max(reps, min(1000, int(40.0 / max(float(pairs.mean()), 1e-3))))):
                fn()

        def in_a_row():          # every result is dropped before the next call, as a caller's loop would
            for _ in range(reps):
                fn()
        T.timed(name, in_a_row)
        cl.synchronize()
        b2b = T.collect()[name][0] / reps
        s = {"avg_ms": round(b2b, 4), "achieved": round(work / (b2b * 1e-3) * scale, 1), "unit": unit,
             "frac_of_peak": round(work / (b2b * 1e-3) * scale / peak, 4), "calls": reps,
             "event_pair_avg_ms": round(float(pairs.mean()), 4), "event_pair_min_ms": round(float(pairs.min()), 4),
             "frac_of_peak_event_pair": round(work / (float(pairs.mean()) * 1e-3) * scale / peak, 4)}
        p = profiled.get("ops", {}).get(name)
        if p:
            s["kernel_only_ms"] = round(p["kernel_us"] * 1e-3, 4)
            s["frac_of_peak_kernel_only"] = round(work / (p["kernel_us"] * 1e-6) * scale / peak, 4)
            if unit == "TFLOP/s":
                s["kernel_only_note"] = "mean of the last %d traced launches after about 40 ms of them" % p.get("kept_calls", 5)
        d[name] = s
    if profiled:
        d["kernel_only_source"] = PROFILE_SUMMARY + " (rocprofv3 --kernel-trace of `bench.py --pmc-configs`, committed)"
    sk = d["c5_addmm_skinny_64x16384x4096"]
    sk["hbm_GBs"] = round(4.0 * (64 * 4096 + 4096 * 16384 + 2 * 64 * 16384) / (sk["avg_ms"] * 1e-3) * 1e-9, 1)
    if "w_addmm_32x16384x4096" in d:   # bound by its long operand's bytes rather than by the matrix cores
        sk = d["w_addmm_32x16384x4096"]
        sk["hbm_GBs"] = round(4.0 * (32 * 4096 + 4096 * 16384 + 2 * 32 * 16384) / (sk["avg_ms"] * 1e-3) * 1e-9, 1)
        sk["frac_of_hbm_peak"] = round(sk["hbm_GBs"] / 8000.0, 4)

    # config 4 as one chain: sumall_gpu + div_gpu + 8 in-place ops, one sync at the end
    pt = cl.ClTensor()
    A = X
    A.copy(cl.ClTensor(oracle.uniform(7, n, 0.0, 1.0)))
    chain = [lambda: A.mul(1.0001), lambda: A.add(0.5), lambda: A.cmul(A), lambda: A.sqrt(), lambda: A.add(pt),
             lambda: A.mul(pt), lambda: A.abs(), lambda: A.csub(0.25)]
    [f() for f in chain[:1]]
    cl.synchronize()
    t0 = time.perf_counter()
    T.timed("c4_chain_10_launches", lambda: [pt.sum(A), A.div(pt)] + [f() for f in chain])
    cl.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    ms = T.collect()["c4_chain_10_launches"]
    d["c4_chain_10_launches"] = {"gpu_ms": round(ms[0], 3), "wall_ms": round(wall, 3),
                                 "achieved": round((4 + 8 * 9) * n / (ms[0] * 1e-3) * 1e-9, 1), "unit": "GB/s",
                                 "note": "sumall_gpu + div_gpu + 8 in-place ops, one sync at the end"}

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
    d["host_copy_GBs"] = host_copy_rates(cl)
    return d


def host_copy_rates(cl, n=1 << 26):
    """Copies of 256 MiB between a tensor and page-locked or ordinary host memory, both directions (best of 3)."""
    from cltorch_amd.tensor import _call
    lib = cl.state().lib
    t = cl.ClTensor(n)
    t.fill(1.0)
    rates = {}
    for name, arr in (("pinned", cl.pinned_array((n,))), ("pageable", np.zeros(n, dtype=np.float32))):
        sz = (C.c_long * 1)(arr.size)
        ft = lib.THFloatTensor_newWithData(arr.ctypes.data_as(C.c_void_p), arr.size, 0, 1, sz, None)
        best = 0.0
        for _ in range(3):
            t0 = time.perf_counter()
            _call("THFloatTensor_copyCl", ft, t._h)
            best = max(best, 4 * n / (time.perf_counter() - t0) * 1e-9)
        rates["d2h_" + name] = round(best, 1)
        best = 0.0
        for _ in range(3):
            t0 = time.perf_counter()
            _call("THClTensor_copyFloat", t._h, ft)
            best = max(best, 4 * n / (time.perf_counter() - t0) * 1e-9)
        rates["h2d_" + name] = round(best, 1)
        lib.THFloatTensor_free(ft)
    return rates


# ------------------------------------------------------------------ profiles ---
PROFILE_SUMMARY = "profiles/bench_pmc_configs_traffic_and_kernel_times.txt"


def committed_profile():
    """The machine-readable line of the committed counter summary (see --summarise), or {}."""
    path = os.path.join(ROOT, PROFILE_SUMMARY)
    if not os.path.exists(path):
        return {}
    for line in open(path):
        if line.startswith("json: "):
            return json.loads(line[6:])
    return {}


def pmc_configs(cl, oracle, n, manifest_path):
    """Launches for hardware-counter and kernel-trace runs over every configuration: a marker (a fill of
    7 elements) opens and closes each operation, which runs 1 + 3 times in between (matrix products 12 to 600 times:
    about 40 ms of launches); the first calls (the first may compile, matrix products start on cool clocks) are dropped
    by the summariser.  The first operation is a dense copy of known size, the calibration point
    of FETCH_SIZE / WRITE_SIZE.  Writes the list of operations with their algorithmic work to
    ``manifest_path``."""
    X, Y, Z = (cl.ClTensor(oracle.uniform(s, n)) for s in (1, 2, 3))
    W = cl.ClTensor(2 * n)
    lo, hi = W.narrow(1, 1, n), W.narrow(1, n + 1, n)
    lo.copy(X)
    pt = cl.ClTensor()
    mk = cl.ClTensor(7)
    ops = [("calibration_copy_2^%d" % int(np.log2(n)), lambda: hi.copy(lo), 8 * n, "GB/s", 3, HBM_PEAK_GBS),
           ("c1_add", lambda: X.add(Y), 12 * n, "GB/s", 3, HBM_PEAK_GBS),
           ("c1_cmul", lambda: X.cmul(Y), 12 * n, "GB/s", 3, HBM_PEAK_GBS),
           ("c1_map2", lambda: X.map2_on_gpu(Y, Z, EXPR), 16 * n, "GB/s", 3, HBM_PEAK_GBS),
           ("c1_sum", lambda: pt.sum(X), 4 * n, "GB/s", 3, HBM_PEAK_GBS),
           ("c1_max", lambda: pt.max(X), 4 * n, "GB/s", 3, HBM_PEAK_GBS)]
    manifest = []

    def run(op):
        name, fn, work, unit, _, peak = op
        # bandwidth kernels: 1 + 3 calls, the mean of the last 3 is kept.  Matrix products: at least 12 calls and about
        # 40 ms of them (the clocks settle over the first tens of ms of such work after a wait), the mean of the last 5
        calls, keep = (4, 3) if unit == "GB/s" else (max(12, min(600, int(40e-3 / (work / (100e12))))), 5)
        mk.fill(0.0)
        for _ in range(calls):
            fn()
        mk.fill(0.0)              # closes the operation: what follows (the next one's set-up) is not part of it
        cl.synchronize()
        manifest.append({"name": name, "work": work, "unit": unit, "peak": peak, "calls": calls, "keep": keep})

    for op in ops:
        run(op)
    del W, lo, hi
    for op in config_ops(cl, oracle, X, Y, Z, n):
        run(op)
    with open(manifest_path, "w") as f:
        json.dump({"elements": n, "ops": manifest}, f)
    print(json.dumps({"pmc_configs": "done", "ops": len(manifest), "manifest": manifest_path}))


def _segments(db_path, want_counters):
    """Dispatches of a rocprofv3 results database in order, per operation (between two one-block FILL markers)."""
    import sqlite3
    c = sqlite3.connect(db_path)
    rows = {}
    if want_counters:
        q = "select dispatch_id, kernel_name, grid_size_x, counter_name, value, duration from counters_collection order by dispatch_id"
        for did, name, gx, cn, v, dur in c.execute(q):
            r = rows.setdefault(did, {"name": name, "gx": gx, "dur": dur, "c": {}})
            r["c"][cn] = r["c"].get(cn, 0.0) + v
    else:
        for did, name, gx, dur in c.execute("select dispatch_id, name, grid_x, duration from kernels order by dispatch_id"):
            rows[did] = {"name": name, "gx": gx, "dur": dur, "c": {}}
    segs, cur = [], None
    for did in sorted(rows):
        r = rows[did]
        if "FILL" in r["name"] and r["gx"] <= 1024:
            cur = []
            segs.append(cur)
        elif cur is not None:
            cur.append(r)
    return segs[0::2]            # a marker opens and another closes every operation: odd segments are set-up in between


def _short(name):
    name = name.replace("void (anonymous namespace)::", "").replace("(anonymous namespace)::", "")
    i = name.find("(")
    return name[:i] if i > 0 else name


WPATH_COUNTERS = ["TCC_EA0_WRREQ_sum", "TCC_EA0_WRREQ_64B_sum", "TCC_EA0_WRREQ_STALL_sum", "TCC_TOO_MANY_EA_WRREQS_STALL_sum",
                  "TCP_TCC_WRITE_REQ_sum", "TCP_TCC_WRITE_REQ_LATENCY_sum"]


def summarise(trace_db, fetch_db, write_db, manifest_path, commands, wpath_db=None):
    """Text summary of three rocprofv3 runs of ``--pmc-configs`` (kernel trace; FETCH_SIZE; WRITE_SIZE), and of a
    fourth with the write-path counters when given."""
    man = json.load(open(manifest_path))
    ops = man["ops"]
    tr, fe, wr = _segments(trace_db, False), _segments(fetch_db, True), _segments(write_db, True)
    assert len(tr) == len(fe) == len(wr) == len(ops), (len(tr), len(fe), len(wr), len(ops))
    wp = _segments(wpath_db, True) if wpath_db else None
    assert wp is None or len(wp) == len(ops)
    out = ["commands (each run from /tmp with TMPDIR=/tmp; $R is the repository root, $OUT a scratch directory):"]
    out += ["  " + c for c in commands]
    out += ["workload: every operation runs 1 + 3 times behind a marker launch; the first call is dropped, the figures are means",
            "  of the other three.  Matrix products (TFLOP/s rows) run 12 times or more (about 40 ms of launches, at most 600) and the",
            "  figures are means of the last five.",
            "  Durations come from the --kernel-trace run (no counters), KiB from the two counter runs.", ""]

    def per_call(seg, op=None):
        calls, keep = (op or {}).get("calls", 4), (op or {}).get("keep", 3)
        assert len(seg) % calls == 0, (len(seg), calls)
        k = len(seg) // calls
        return k, seg[k * (calls - keep):]          # the kept calls

    # calibration on the dense copy: reads and writes 4 bytes per element
    k, cal_f = per_call(fe[0], ops[0])
    _, cal_w = per_call(wr[0], ops[0])
    n = man["elements"]
    want_kib = 4.0 * n / 1024
    f_read = sum(r["c"].get("FETCH_SIZE", 0.0) for r in cal_f) / (len(cal_f) / k)
    w_read = sum(r["c"].get("WRITE_SIZE", 0.0) for r in cal_w) / (len(cal_w) / k)
    fs, ws = want_kib / f_read, want_kib / w_read
    out += [f"calibration: {_short(cal_f[0]['name'])} on 2^{int(np.log2(n))} elements reads {want_kib:.0f} KiB and writes {want_kib:.0f} KiB;",
            f"  FETCH_SIZE reports {f_read:.1f} KiB -> scale {fs:.4f}; WRITE_SIZE reports {w_read:.1f} KiB -> scale {ws:.4f}", ""]
    hdr = "%-34s %-44s %3s %9s %11s %11s %9s %9s %7s %7s" % ("operation", "kernel", "x", "dur_us", "FETCH_KiB", "WRITE_KiB", "read_MiB",
                                                               "wrote_MiB", "traf/alg", "frac")
    if wp:
        hdr += " %10s %9s %9s" % ("wr_req", "stall/req", "lat/req")
    out += [hdr, "-" * len(hdr)]
    js = {"elements": n, "fetch_scale": round(fs, 4), "write_scale": round(ws, 4), "ops": {}}
    for idx, (op, st, sf, sw) in enumerate(zip(ops, tr, fe, wr)):
        k, t = per_call(st, op)
        _, f = per_call(sf, op)
        _, w = per_call(sw, op)
        wpc = per_call(wp[idx], op)[1] if wp else None
        ncalls = len(t) // k if k else 0
        if not k:
            out.append("%-34s (no device kernel)" % op["name"])
            continue
        tot_us = tot_rd = tot_wr = 0.0
        lines = []
        for j in range(k):         # j-th kernel of each call
            us = np.mean([t[i * k + j]["dur"] for i in range(ncalls)]) / 1e3
            fk = np.mean([f[i * k + j]["c"].get("FETCH_SIZE", 0.0) for i in range(ncalls)])
            wk = np.mean([w[i * k + j]["c"].get("WRITE_SIZE", 0.0) for i in range(ncalls)])
            tot_us += us
            tot_rd += fk * fs * 1024
            tot_wr += wk * ws * 1024
            lines.append((_short(t[j]["name"])[:44], us, fk, wk))
        is_bw = op["unit"] == "GB/s"
        ratio = (tot_rd + tot_wr) / op["work"] if is_bw else None
        frac = op["work"] / (tot_us * 1e-6) * (1e-9 if is_bw else 1e-12) / op["peak"]
        for j, (kn, us, fk, wk) in enumerate(lines):
            first = j == 0
            line = "%-34s %-44s %3s %9.1f %11.1f %11.1f %9s %9s %7s %7s" % (
                op["name"][:34] if first else "", kn, "", us, fk, wk,
                "%.1f" % (tot_rd / 2 ** 20) if first else "", "%.1f" % (tot_wr / 2 ** 20) if first else "",
                ("%.3f" % ratio if ratio is not None else "-") if first else "", "%.3f" % frac if first else "")
            if wpc and len(wpc) == len(t):
                cnt = lambda name: float(np.mean([wpc[i * k + j]["c"].get(name, 0.0) for i in range(ncalls)]))
                req, tcp = cnt("TCC_EA0_WRREQ_sum"), cnt("TCP_TCC_WRITE_REQ_sum")
                line += " %10.4g %9s %9s" % (req, "%.2f" % (cnt("TCC_EA0_WRREQ_STALL_sum") / req) if req > 1e4 else "-",
                                             "%.0f" % (cnt("TCP_TCC_WRITE_REQ_LATENCY_sum") / tcp) if tcp > 1e4 else "-")
            out.append(line)
        js["ops"][op["name"]] = {"kernel_us": round(tot_us, 2), "read_bytes": int(tot_rd), "written_bytes": int(tot_wr),
                                 "work": op["work"], "unit": op["unit"], "frac": round(frac, 4), "kept_calls": ncalls}
    out += ["", "columns: dur_us = mean kernel duration; FETCH/WRITE_KiB = counter values per dispatch; read/wrote_MiB = scaled HBM bytes of one call;",
            "  traf/alg = (read + written) / algorithmic bytes of the call; frac = algorithmic work / kernel time / peak (8000 GB/s or 157.3 TFLOP/s).",
            "  wr_req = write requests of the L2s to memory per dispatch (TCC_EA0_WRREQ_sum; all of 64 bytes in every row here);",
            "  stall/req = TCC_EA0_WRREQ_STALL_sum / wr_req (cycles a request waited for credits on its way out of the L2);",
            "  lat/req = TCP_TCC_WRITE_REQ_LATENCY_sum / TCP_TCC_WRITE_REQ_sum (cycles from a vector cache's write request to its acknowledgement).",
            "json: " + json.dumps(js)]
    return "\n".join(out) + "\n"


def summarise_trace(db_path):
    """Per-kernel totals of a `rocprofv3 --kernel-trace --stats -- python3 bench.py` run."""
    import sqlite3
    c = sqlite3.connect(db_path)
    rows = list(c.execute("select name, total_calls, total_duration, average, percentage from top_kernels"))
    extra = {}
    for name, mn, mx, vg, lds in c.execute("select name, min(duration), max(duration), max(vgpr_count), max(lds_size) from kernels group by name"):
        extra[name] = (mn, mx, vg, lds)
    out = ["command (run from /tmp with TMPDIR=/tmp; $R is the repository root, $OUT a scratch directory):",
           "  rocprofv3 --kernel-trace --stats -d $OUT/bench_trace -o b -- python3 $R/bench.py --no-cpu",
           "  python3 bench.py --summarise-trace $OUT/bench_trace/b_results.db > profiles/bench_all_configs_kernel_trace.txt",
           "source: view top_kernels of the results database; durations in microseconds", "",
           "%-84s %6s %12s %10s %10s %10s %6s %6s %7s" % ("kernel", "calls", "total_us", "avg_us", "min_us", "max_us", "pct", "vgpr", "lds")]
    for name, calls, tot, avg, pct in rows:
        mn, mx, vg, lds = extra.get(name, (0, 0, 0, 0))
        out.append("%-84s %6d %12.1f %10.1f %10.1f %10.1f %6.2f %6s %7s" % (_short(name)[:84], calls, tot, avg, mn / 1e3, mx / 1e3, pct, vg, lds))
    return "\n".join(out) + "\n"


def summarise_mfma(db_path):
    """Matrix-core duty of the addmm launches of ``--pmc-gemm`` from one counter run."""
    import sqlite3
    c = sqlite3.connect(db_path)
    rows = {}
    q = "select dispatch_id, kernel_name, grid_size_x, grid_size_y, counter_name, value, duration from counters_collection order by dispatch_id"
    for did, name, gx, gy, cn, v, dur in c.execute(q):
        r = rows.setdefault(did, {"name": name, "gx": gx, "gy": gy, "dur": dur, "c": {}})
        r["c"][cn] = r["c"].get(cn, 0.0) + v
    out = ["command (run from /tmp with TMPDIR=/tmp; $R is the repository root, $OUT a scratch directory):",
           "  rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE --kernel-trace -d $OUT/pmc_gemm -o g -- python3 $R/bench.py --pmc-gemm",
           "  python3 bench.py --summarise-mfma $OUT/pmc_gemm/g_results.db > profiles/addmm_8192_and_skinny_pmc_mfma_duty.txt",
           "workload: addmm 8192^3 five times, addmm 64x16384x4096 (A given transposed) 600 times, then 4095^3 and 3000x5000x7000",
           "  12 times each (their last three launches are listed); fp32, random normal operands", "",
           "how to read it: every v_mfma_f32_32x32x2_f32 books 64 busy cycles on its SIMD, so flops = busy / 64 * 4096;",
           "  duty = SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs * GRBM_GUI_ACTIVE / 8 XCDs); clock = GRBM_GUI_ACTIVE / 8 / duration.",
           "  For kernels shorter than ~0.2 ms GRBM_GUI_ACTIVE also covers some time around the launch, so their clock reads a little",
           "  high and their duty a little low.  Of the 600 skinny launches every hundredth is listed.", "",
           "%-52s %10s %8s %14s %14s %8s %10s %8s" % ("kernel", "grid", "dur_us", "MFMA_BUSY", "GRBM_ACTIVE", "duty", "clock_GHz", "TFLOP/s")]
    total, seen = {}, {}
    for r in rows.values():
        if "gemm" in r["name"]:
            total[_short(r["name"])] = total.get(_short(r["name"]), 0) + 1
    for did in sorted(rows):
        r = rows[did]
        if "gemm" not in r["name"]:
            continue
        key = _short(r["name"])
        seen[key] = seen.get(key, 0) + 1
        # kernels launched a few times: all of the square product's five, else the last three; the 600: every hundredth
        if total[key] > 20 and seen[key] % 100:
            continue
        if 5 < total[key] <= 20 and seen[key] <= total[key] - 3:
            continue
        busy, act = r["c"].get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0), max(r["c"].get("GRBM_GUI_ACTIVE", 1.0), 1.0)
        flops = busy / 64.0 * 4096.0
        out.append("%-52s %10s %8.1f %14.4g %14.4g %8.3f %10.2f %8.1f" % (
            key[:52], "%dx%d" % (r["gx"] // 256, r["gy"]), r["dur"] / 1e3, busy, act, busy / 1024.0 / (act / 8.0), act / 8.0 / r["dur"],
            flops / r["dur"] / 1e3))
    return "\n".join(out) + "\n"


if __name__ == "__main__":
    main()
