#!/usr/bin/env python3
"""Throughput of the HIP skeletons on one MI355X, on the five benchmark
configurations, with inputs already resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME]] [--no-cpu]

A step is one pass of a skeleton over its full-size synthetic input (for the
iterated stencil: the ten applications).  The headline line is the prefix sum
`scanl (+) 0` over 2^26 Int32; the other configurations are reported under
"skeletons" in the same JSON line.  One GPU only.

Consecutive steps work on DIFFERENT copies of the input and different result
buffers (--sets of them, used round robin, together several times the 256 MB
of the memory-side cache), so that no step finds the previous step's data in a
cache: the figures are those of data that comes from and goes to HBM.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "accelerate-cuda_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0


def log(*a):
    print(*a, file=sys.stderr)
    sys.stderr.flush()


class Timer(object):
    """W warm-up steps, then exactly K timed steps: wall clock between two
    device synchronisations, and HIP events recorded on the launch stream."""

    DEVICE_WARMUP_MS = 60.0       # before the first warm-up step of a run that finds the device idle: it leaves its idle clocks
    IDLE_AFTER_S = 0.25           # (idle = nothing launched for this long: process start, a CPU leg, building inputs)

    def __init__(self, A, ctx, stream, steps, warmup):
        self.A, self.ctx, self.stream, self.steps, self.warmup = A, ctx, stream, steps, warmup
        self.e0, self.e1 = ctx.event(True), ctx.event(True)
        self.last_busy = None

    def run(self, step):
        """`step` is one callable, or a list of them (one per buffer set) taken round robin"""
        steps = step if isinstance(step, (list, tuple)) else [step]
        k = 0
        if self.last_busy is None or time.perf_counter() - self.last_busy > self.IDLE_AFTER_S:
            # (the first call of a step may build a variant of its instance -- seconds of compilation on a machine
            # with cold caches -- which must not count as time the device was kept busy)
            steps[0]()
            k += 1
            self.ctx.sync()
            t_end = time.perf_counter() + self.DEVICE_WARMUP_MS * 1e-3
            while time.perf_counter() < t_end:
                for _ in range(16):
                    steps[k % len(steps)]()
                    k += 1
                self.ctx.sync()
        for _ in range(max(self.warmup, len(steps))):
            steps[k % len(steps)]()
            k += 1
        self.ctx.sync()
        t0 = time.perf_counter()
        self.ctx.record(self.e0, self.stream)
        for _ in range(self.steps):
            steps[k % len(steps)]()
            k += 1
        self.ctx.record(self.e1, self.stream)
        self.ctx.sync()
        wall_ms = (time.perf_counter() - t0) * 1e3 / self.steps
        event_ms = self.ctx.elapsed_ms(self.e0, self.e1) / self.steps
        self.last_busy = time.perf_counter()
        return wall_ms, event_ms


def cpu_leg(fn, what, bytes_per_call, budget_s=3.0):
    """the oracle's restatement of the reference's algorithm, one thread, timed for about `budget_s` seconds"""
    reps, t0 = 0, time.perf_counter()
    while reps == 0 or time.perf_counter() - t0 < budget_s:
        fn()
        reps += 1
    per = (time.perf_counter() - t0) / reps
    return {"value": round(bytes_per_call / per / 1e9, 3), "unit": "GB/s", "ms_per_step": round(per * 1e3, 3), "cores": 1, "kind": "port",
            "sample": "%s, %d repetition(s), 1 thread of %d host cores; an upper bound on the boxed Haskell interpreter"
                      % (what, reps, os.cpu_count())}


def end_to_end(ctx, uploads, run, download, reps=3):
    """what the reference's `run1` does around its kernels (CUDA.hs:382-389, Execute.hs:146-154): the operands go from
    pageable host memory to the device, the kernels run, the result comes back into pageable host memory.  `uploads`
    pairs device arrays with the host arrays they take; best of `reps`.  Timed twice: with the library's staged
    transfers (pinned buffers of its own, chunks copied by a few threads while the copy engine moves the chunks before
    them), and with the runtime's own copies from and to pageable memory (a second context with `copy.staged=0`)."""
    import acchip as A
    L = A.lib()
    if getattr(end_to_end, "skip", False):
        return None
    plain = getattr(end_to_end, "plain", None)
    if plain is None:
        with A.tuning("copy.staged=0"):
            plain = end_to_end.plain = A.Context(ctx.device)
    first = download.get()
    host_out = np.empty_like(first)
    host_out[...] = 0                               # its pages exist: the timed copies do not pay for their first touch
    res = {}
    for name, handle in (("staged", ctx.handle), ("runtime_pageable", plain.handle)):
        best = None
        for _ in range(reps):
            ctx.sync()
            t0 = time.perf_counter()
            for d, h in uploads:
                A.check(L.acc_memcpy_h2d(handle, d.ptr, h.ctypes.data_as(C.c_void_p), h.nbytes))
            run()
            src = download.where() if hasattr(download, "where") else download
            A.check(L.acc_stream_sync(ctx.handle, end_to_end.stream))
            A.check(L.acc_memcpy_d2h(handle, host_out.ctypes.data_as(C.c_void_p), src.ptr, src.nbytes))
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        res[name] = best
    assert np.array_equal(host_out, download.get()), "end to end: the staged and the plain copy disagree"
    moved = sum(h.nbytes for _, h in uploads) + host_out.nbytes
    return {"ms": round(res["staged"] * 1e3, 3), "host_bytes_moved": int(moved),
            "GB_per_s_over_the_link": round(moved / res["staged"] / 1e9, 2),
            "runtime_pageable_ms": round(res["runtime_pageable"] * 1e3, 3),
            "runtime_pageable_GB_per_s": round(moved / res["runtime_pageable"] / 1e9, 2),
            "note": "H2D of the operands from pageable memory + kernels + D2H of the result into pageable memory, device buffers reused; not the headline"}


def kernel_sources_hash():
    """SHA-256 over what decides the code of every kernel: the device templates and the generator.  The profile
    summaries under profiles/ carry the hash of the tree they were measured on; a summary whose hash is not the
    tree's describes other kernels than the ones this run launches."""
    import glob
    import hashlib
    csrc = os.path.join(ROOT, "accelerate-cuda_amd", "csrc")
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(csrc, "device", "*.h"))) + [os.path.join(csrc, "skeleton.cpp")]:
        h.update(os.path.basename(path).encode() + b"\0")
        h.update(open(path, "rb").read())
    return h.hexdigest()


def profile_hash(path):
    """the `kernel-sources-sha256:` line of a profile summary, or None"""
    try:
        for line in open(path):
            if line.startswith("kernel-sources-sha256:"):
                return line.split()[1]
    except OSError:
        pass
    return None


def profiled_traffic(kernel):
    """HBM bytes per launch of `kernel` as rocprofv3 counted them (FETCH_SIZE and WRITE_SIZE, each scaled by what the
    same counter reads for a plain copy of known size): read from the committed summary, not measured in this run;
    `stale` says whether the summary was measured on other kernel sources than this tree's"""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.txt")
    try:
        for line in open(path):
            f = line.split()
            if len(f) >= 3 and f[0] == "traffic" and f[1] == kernel:
                measured_on = profile_hash(path)
                return {"bytes": int(float(f[2])), "source": "profiles/hbm_traffic_per_launch.txt",
                        "kernel_sources_sha256": measured_on, "stale": measured_on != kernel_sources_hash()}
    except OSError:
        pass
    return None


def result(name, wall_ms, event_ms, launches_per_step, bytes_per_launch, elements_per_step, extra=None):
    launch_ms = event_ms / launches_per_step
    gbs = bytes_per_launch / (launch_ms * 1e-3) / 1e9
    r = {"ms_per_step": round(wall_ms, 5), "event_ms_per_step": round(event_ms, 5),
         "kernel_launches_per_step": launches_per_step, "avg_launch_us": round(launch_ms * 1e3, 3),
         "algorithmic_bytes_per_launch": int(bytes_per_launch), "GB_per_s": round(gbs, 1),
         "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
         "elements_per_s": round(elements_per_step / (event_ms * 1e-3), 1)}
    if extra:
        r.update(extra)
    t = profiled_traffic(r.pop("traffic_key", None))
    if t:
        r["hbm_traffic_bytes"], r["hbm_traffic_source"] = t["bytes"], t["source"]
        r["hbm_traffic_stale"] = t["stale"]
        r["traffic_over_algorithmic"] = round(t["bytes"] / float(bytes_per_launch), 3)
    log("  %-28s %9.3f us/launch  %8.1f GB/s  %5.1f%% of HBM peak" % (name, launch_ms * 1e3, gbs, 100 * gbs / HBM_PEAK_GBS))
    return r


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--only", type=str, default="")
    ap.add_argument("--sets", type=int, default=4, help="copies of every configuration's buffers, used round robin")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--plain", action="store_true",
                    help="only the warm-up and the timed steps of every configuration: no one-by-one, end-to-end or CPU legs "
                         "(a counter run then sees a known number of dispatches per kernel)")
    ap.add_argument("--kernel-sources-hash", action="store_true", help="print the hash the profile summaries are tied to, and leave")
    ap.add_argument("--device-warmup-ms", type=float, default=Timer.DEVICE_WARMUP_MS,
                    help="untimed launches before the warm-up steps of a configuration that finds the device idle")
    args = ap.parse_args()
    if args.kernel_sources_hash:
        print(kernel_sources_hash())
        return
    Timer.DEVICE_WARMUP_MS = args.device_warmup_ms
    if args.plain:
        args.no_cpu = True
        Timer.IDLE_AFTER_S = -1.0             # every configuration starts with its first call on its own: the same number of dispatches each
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)" % args.gpus)

    import acchip as A
    import workloads as wl

    only = set(s for s in args.only.split(",") if s)
    want = lambda name: (not only) or name in only   # noqa: E731

    ctx = A.Context(0)
    props = ctx.props()
    log("device: arch %s, %d CUs, LDS/workgroup %d, L2 %d" % (props.arch.decode(), props.compute_units, props.lds_per_block, props.l2_bytes))
    stream = ctx.stream()
    end_to_end.stream = stream
    end_to_end.skip = args.plain
    T = Timer(A, ctx, stream, args.steps, args.warmup)

    def traced(steps, calls=12):
        """the same launches one by one onto an idle device, an event before and behind each (acc_trace_start/stop):
        the way the front-end leg below is timed, for the figure its calls are to be held against"""
        if args.plain:
            return None
        ctx.sync()
        ctx.trace_start()
        for k in range(calls):
            steps[k % len(steps)]()
            ctx.sync()
        launches, ms = ctx.trace_stop()
        return round(ms * 1e3 / calls, 3)
    L = A.lib()
    F32, I32 = (1, "float"), (1, "Int32")
    sk = {}
    headline = None
    S = max(1, args.sets)

    def rd(k):
        """fragment text for a linear read of input k at ix"""
        return ("acc_stream(arrIn%d_0, ix)" if os.environ.get("ACC_BENCH_STREAM", "1") == "1" else "arrIn%d_0[ix]") % k

    def envs(*arrs):
        e = (A.acc_array * len(arrs))()
        for k, a in enumerate(arrs):
            e[k] = a.desc()
        return e

    # ---------------------------------------------------------------- 2: prefix sums
    n = 1 << 26
    if want("scan"):
        log("prefix sums over 2^26 Int32 ...")
        x = wl.scan_input(n)
        dxs = [ctx.array(x) for _ in range(S)]
        env_s = [envs(d) for d in dxs]
        outs = [ctx.empty(n + 1, np.int32) for _ in range(S)]
        for kind in ("scanl", "scanl1", "scanr"):
            s = ctx.skeleton(A.SCAN_KINDS[kind], "Int32", env=[I32], get=rd(0),
                             combine="x + y", seed=None if kind == "scanl1" else "0")
            ods = [o.desc(shape=(n + (0 if kind == "scanl1" else 1),)) for o in outs]

            def step(i, s=s, ods=ods):
                return lambda: A.check(L.acc_exec_scan(s.handle, env_s[i], n, C.byref(ods[i]), None, stream))
            w, e = T.run([step(i) for i in range(S)])
            sk[kind] = result(kind + " (+) Int32 2^26", w, e, 1, 2 * n * 4 + 4, n, {"traffic_key": kind})
            if kind == "scanl":
                sk[kind]["one_by_one_us"] = traced([step(i) for i in range(S)])
                sk[kind]["end_to_end"] = end_to_end(ctx, [(dxs[0], x)], step(0), outs[0])
                headline = dict(sk[kind], wall_ms=w, event_ms=e)
                # size-independent check: the last element is the sum, the first the seed
                got = outs[S - 1].get()
                if os.environ.get("ACC_BENCH_NOCHECK"):
                    continue
                assert int(got[0]) == 0 and int(got[-1]) == int(x.sum(dtype=np.int64)), "scanl total mismatch"
                assert np.array_equal(np.diff(got), x), "scanl increments mismatch"
        if not args.no_cpu:
            from oracle import oracle as orc
            orc.build()
            reps, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < 10.0:
                orc.scan("scanl", orc.OP_ADD, x, seed=0)
                reps += 1
            cpu_s = (time.perf_counter() - t0) / reps
            cpu = {"value": round((2 * n * 4 + 4) / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                   "sample": "oracle/acc_oracle.c orc_scan_i32 (scanl), full 2^26-element input, %d repetitions, "
                             "1 thread of %d host cores; an upper bound on the boxed Haskell interpreter" % (reps, os.cpu_count())}
        else:
            cpu = None
        del dxs, outs, env_s, x
    else:
        cpu = None

    # ---------------------------------------------------------------- map family (calibration: a plain copy)
    if want("map"):
        log("map: copy and zipWith (*) over 2^26 elements ...")
        x = wl.scan_input(n)
        dxs, outs = [ctx.array(x) for _ in range(S)], [ctx.empty(n, np.int32) for _ in range(S)]
        env_s = [envs(d) for d in dxs]
        cp = ctx.skeleton(A.SKEL_MAP, "Int32", env=[I32], out_rank=1, get=rd(0))
        ods = [o.desc() for o in outs]

        def step(i):
            return lambda: A.check(L.acc_exec_map(cp.handle, env_s[i], C.byref(ods[i]), stream))
        w, e = T.run([step(i) for i in range(S)])
        assert np.array_equal(outs[S - 1].get(), x)
        sk["map_copy"] = result("map id Int32 2^26 (copy)", w, e, 1, 2 * n * 4, n, {"traffic_key": "map_copy"})
        del dxs, outs, env_s
        fx = x.astype(np.float32)
        fy = fx[::-1].copy()
        dfx, dfy, fo = [ctx.array(fx) for _ in range(S)], [ctx.array(fy) for _ in range(S)], [ctx.empty(n, np.float32) for _ in range(S)]
        env2 = [envs(dfx[i], dfy[i]) for i in range(S)]
        zw = ctx.skeleton(A.SKEL_MAP, "float", env=[F32, F32], out_rank=1, get=rd(0) + " * " + rd(1))
        fod = [o.desc() for o in fo]

        def step(i):
            return lambda: A.check(L.acc_exec_map(zw.handle, env2[i], C.byref(fod[i]), stream))
        w, e = T.run([step(i) for i in range(S)])
        assert np.array_equal(fo[S - 1].get(), fx * fy)
        sk["zipwith_mul"] = result("zipWith (*) Float32 2^26", w, e, 1, 3 * n * 4, n)
        sk["zipwith_mul"]["end_to_end"] = end_to_end(ctx, [(dfx[0], fx), (dfy[0], fy)], step(0), fo[0])
        if not args.no_cpu:
            from oracle import oracle as orc
            orc.build()
            sk["zipwith_mul"]["cpu_baseline"] = cpu_leg(lambda: orc.zipwith_mul_f32(fx, fy), "oracle/acc_oracle.c orc_zipwith_mul_f32, full 2^26 elements", 3 * n * 4)
        del dfx, dfy, fo, env2, x, fx, fy

    # ---------------------------------------------------------------- 1: dot product
    if want("dot"):
        log("dot product of two 2^24 Float32 vectors ...")
        nd = 1 << 24
        x, y = wl.dot_inputs(nd)
        Sd = 4 * S                                  # 128 MB per set: more sets to get past the cache
        dxs, dys = [ctx.array(x) for _ in range(Sd)], [ctx.array(y) for _ in range(Sd)]
        env_s = [envs(dxs[i], dys[i]) for i in range(Sd)]
        dot = ctx.skeleton(A.SKEL_FOLD, "float", env=[F32, F32], out_rank=0, get=rd(0) + " * " + rd(1),
                           combine="x + y", seed="0.0f")
        o = ctx.empty((), np.float32)
        od = o.desc()
        sh = (C.c_int64 * 1)(nd)

        def step(i):
            return lambda: A.check(L.acc_exec_fold(dot.handle, env_s[i], 1, sh, C.byref(od), stream))
        w, e = T.run([step(i) for i in range(Sd)])
        dot_one_by_one = traced([step(i) for i in range(Sd)])
        truth = float((x.astype(np.float64) * y.astype(np.float64)).sum())     # (not np.dot: its BLAS threads keep spinning for milliseconds and would take the cores from the copies of the end-to-end leg)
        sk["dot"] = result("fold (+) 0 . zipWith (*) 2^24", w, e, 1, 2 * nd * 4 + 4, nd,
                           {"result": float(o.get()), "float64_truth": truth, "GFLOP_per_s": round(2 * nd / (e * 1e-3) / 1e9, 1),
                            "traffic_key": "foldAll", "one_by_one_us": dot_one_by_one})
        sk["dot"]["end_to_end"] = end_to_end(ctx, [(dxs[0], x), (dys[0], y)], step(0), o)
        if not args.no_cpu:
            from oracle import oracle as orc
            orc.build()
            sk["dot"]["cpu_baseline"] = cpu_leg(lambda: orc.dot_f32(x, y), "oracle/acc_oracle.c orc_dot_f32, full 2^24 elements", 2 * nd * 4 + 4)
        del dxs, dys, env_s

    # ---------------------------------------------------------------- 3: histograms
    for name, bins, gen in (("hist256_uniform", 256, wl.hist_uniform_keys), ("hist65536_zipf", 65536, wl.hist_zipf_keys)):
        if not want(name) and not want("hist"):
            continue
        log("histogram %s over 2^26 Int32 keys ..." % name)
        keys = gen(n, bins)
        dks = [ctx.array(keys) for _ in range(S)]
        env_s = [envs(d) for d in dks]
        hist = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y",
                            permutation=rd(0), combine_hint=A.COMBINE_ADD)
        dfl, out = ctx.array(np.zeros(bins, np.int32)), ctx.empty(bins, np.int32)
        dd, od = dfl.desc(), out.desc()

        def step(i):
            return lambda: A.check(L.acc_exec_permute(hist.handle, env_s[i], n, C.byref(dd), C.byref(od), stream))
        w, e = T.run([step(i) for i in range(S)])
        got = out.get()
        assert os.environ.get("ACC_BENCH_NOCHECK") or (int(got.sum()) == n and np.array_equal(got, np.bincount(keys, minlength=bins))), "histogram mismatch"
        sk[name] = result("permute (+) %d bins" % bins, w, e, 1, n * 4 + 2 * bins * 4, n,
                          {"Gkeys_per_s": round(n / (e * 1e-3) / 1e9, 2), "note": "step = every launch the call makes: one kernel (256 bins: its first workgroup copies the defaults); main kernel + merge (65 536 bins)",
                           "traffic_key": name})
        sk[name]["end_to_end"] = end_to_end(ctx, [(dks[0], keys)], step(0), out)
        if not args.no_cpu:
            from oracle import oracle as orc
            orc.build()
            zeros = np.zeros(bins, np.int32)
            sk[name]["cpu_baseline"] = cpu_leg(lambda: orc.permute(orc.OP_ADD, zeros, keys), "oracle/acc_oracle.c orc_permute_i32 (source = 1), full 2^26 keys",
                                               n * 4 + 2 * bins * 4)
        del dks, env_s, keys

    # ---------------------------------------------------------------- 4: stencils
    if want("stencil"):
        log("3x3 Gaussian (clamp) x10 and 5-point Laplacian (mirror) on 8192x8192 Float32 ...")
        h = w_ = 8192
        img = wl.stencil_image(h, w_)
        a_s, b_s = [ctx.array(img) for _ in range(S)], [ctx.empty((h, w_), np.float32) for _ in range(S)]
        ad, bd = [a.desc() for a in a_s], [b.desc() for b in b_s]
        taps = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
        gauss = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=taps, boundary="clamp",
                             stencil_fn=A.linear_stencil_fn([1, 2, 1, 2, 4, 2, 1, 2, 1], 16))
        lap = ctx.skeleton(A.SKEL_STENCIL, "float", out_rank=2, taps=[(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)],
                           boundary="mirror", stencil_fn=A.linear_stencil_fn([1, 1, -4, 1, 1]))
        rib = C.c_int32(0)

        def step(i):
            return lambda: A.check(L.acc_exec_stencil_iterate(gauss.handle, None, C.byref(ad[i]), C.byref(bd[i]), 10, stream, C.byref(rib)))
        w, e = T.run([step(i) for i in range(S)])
        sk["gaussian3x3_clamp_x10"] = result("stencil 3x3 gaussian x10", w, e, 10, 2 * h * w_ * 4, 10 * h * w_, {"traffic_key": "stencil_gaussian"})

        class _where(object):              # the result of the ten applications lies in a or in b
            @staticmethod
            def where():
                return b_s[0] if rib.value else a_s[0]

            @staticmethod
            def get():
                return _where.where().get()
        sk["gaussian3x3_clamp_x10"]["end_to_end"] = end_to_end(ctx, [(a_s[0], img)], step(0), _where)
        if not args.no_cpu:
            from oracle import oracle as orc
            orc.build()
            g_taps = [(dy, dx, c) for (dy, dx), c in zip(taps, [1, 2, 1, 2, 4, 2, 1, 2, 1])]
            sk["gaussian3x3_clamp_x10"]["cpu_baseline"] = cpu_leg(
                lambda: orc.stencil2d(img, g_taps, 16.0, "clamp", iters=1),
                "oracle/acc_oracle.c orc_stencil2d_iter_f32, ONE of the ten applications on the full 8192x8192 image (figures per application)",
                2 * h * w_ * 4, budget_s=2.0)

        def step2(i):
            return lambda: A.check(L.acc_exec_stencil(lap.handle, None, C.byref(ad[i]), C.byref(bd[i]), stream))
        w, e = T.run([step2(i) for i in range(S)])
        sk["laplace5_mirror"] = result("stencil 5-point laplacian", w, e, 1, 2 * h * w_ * 4, h * w_, {"traffic_key": "stencil_laplace"})
        del a_s, b_s, img

    # ---------------------------------------------------------------- 5: sparse matrix-vector product
    if want("smvm"):
        log("CSR SMVM, 2^20 rows, Poisson(32) row lengths ...")
        vals, cols, offs, lens, xv = wl.smvm_inputs()
        nnz, rows = vals.size, offs.size - 1
        dv, dc = [ctx.array(vals) for _ in range(S)], [ctx.array(cols) for _ in range(S)]
        dxv, doff = [ctx.array(xv) for _ in range(S)], [ctx.array(offs) for _ in range(S)]
        env_s = [envs(dv[i], dc[i], dxv[i]) for i in range(S)]
        ys = [ctx.empty(rows, np.float32) for _ in range(S)]
        smvm = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[F32, I32, F32],
                            get=os.environ.get("ACC_BENCH_SMVM_GET", rd(0) + " * arrIn2_0[" + rd(1) + "]"),
                            combine="x + y", seed="0.0f")
        offd, yd = [d.desc() for d in doff], [y.desc() for y in ys]

        def step(i):
            return lambda: A.check(L.acc_exec_foldseg(smvm.handle, env_s[i], nnz, C.byref(offd[i]), C.byref(yd[i]), stream))
        w, e = T.run([step(i) for i in range(S)])
        smvm_one_by_one = traced([step(i) for i in range(S)])
        y = ys[S - 1]
        sk["smvm"] = result("foldSeg (+) . zipWith (*) . gather", w, e, 1, nnz * 8 + rows * 8 + xv.size * 4, nnz,
                            {"nnz": int(nnz), "GFLOP_per_s": round(2 * nnz / (e * 1e-3) / 1e9, 1),
                             "note": "segment offsets precomputed on the device (scanl over the 2^20 lengths is not in the step)",
                             "traffic_key": "foldSeg", "one_by_one_us": smvm_one_by_one})
        # composition check on the device result: y = A x in float64 within 1e-4 of the row's magnitude
        import scipy.sparse as sp
        Amat = sp.csr_matrix((vals.astype(np.float64), cols, offs), shape=(rows, xv.size))
        truth = Amat @ xv.astype(np.float64)
        mag = abs(Amat) @ np.abs(xv.astype(np.float64))
        assert np.all(np.abs(y.get() - truth) <= 1e-4 * np.maximum(np.abs(truth), 1e-3 * mag) + 1e-30), "smvm mismatch"
        # What bounds it: the same kernel with the product left out (the gather of x alone: one request to the L2 per
        # non-zero, whatever else the kernel does) and with the gather replaced by a linear read (the kernel's own
        # structure at the speed of a stream).  The L2s answer a request per channel and clock at best:
        # 8 XCDs x 16 channels x the L2 clock; the gathers are held against that.
        legs = {}
        for leg, get in (("gather_only", "arrIn2_0[" + rd(1) + "]"), ("linear_read_instead_of_gather", rd(0) + " * (float)" + rd(1))):
            sk_leg = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[F32, I32, F32], get=get, combine="x + y", seed="0.0f")

            def step_leg(i, sk_leg=sk_leg):
                return lambda: A.check(L.acc_exec_foldseg(sk_leg.handle, env_s[i], nnz, C.byref(offd[i]), C.byref(yd[i]), stream))
            wl_, el_ = T.run([step_leg(i) for i in range(S)])
            legs[leg] = round(el_ * 1e3, 3)
            log("  %-28s %9.3f us/launch" % ("smvm, " + leg.replace("_", " "), el_ * 1e3))
        l2_clock_ghz = 2.1                                  # the L2s' clock on this part (the shader clock is 2.4 GHz at its peak)
        req_peak = 8 * 16 * l2_clock_ghz * 1e9              # requests a second at one a channel and clock
        req_rate = nnz / (sk["smvm"]["avg_launch_us"] * 1e-6)
        sk["smvm"].update({
            "gather_floor_us": legs["gather_only"], "linear_read_us": legs["linear_read_instead_of_gather"],
            "over_gather_floor": round(sk["smvm"]["avg_launch_us"] / legs["gather_only"], 3),
            "roofline_l2_requests": {"bound": "l2_requests", "achieved": round(req_rate / 1e9, 1), "peak": round(req_peak / 1e9, 1),
                                     "unit": "G requests/s", "frac": round(req_rate / req_peak, 3),
                                     "note": "one 4-byte gather of x per non-zero = one request to an L2 channel; peak = 8 XCDs x 16 channels x %.1f GHz" % l2_clock_ghz}})
        sk["smvm"]["end_to_end"] = end_to_end(ctx, [(dv[0], vals), (dc[0], cols), (dxv[0], xv), (doff[0], offs)], step(0), ys[0])
        if not args.no_cpu:
            from oracle import oracle as orc
            orc.build()
            sk["smvm"]["cpu_baseline"] = cpu_leg(lambda: orc.smvm_f32(vals, cols, offs, xv), "oracle/acc_oracle.c orc_smvm_f32, full 2^20 rows",
                                                 nnz * 8 + rows * 8 + xv.size * 4)
    # ---------------------------------------------------------------- what a first `run` costs, and what a call costs the host
    if want("startup"):
        log("start-up: compilation cold, from the disk cache, from memory; two kernels one after the other and side by side ...")
        nonce = "// %d.%d" % (os.getpid(), time.time_ns())
        st = {}

        def build(name, k, wait=True, **kw):
            t0 = time.perf_counter()
            skx = ctx.skeleton(*kw.pop("args"), preamble="%s %s %d" % (nonce, name, k), wait=wait, **kw)
            return skx, (time.perf_counter() - t0) * 1e3
        kinds = {
            "scanl": dict(args=(A.SKEL_SCANL, "Int32"), env=[I32], get=rd(0), combine="x + y", seed="0"),
            "dot": dict(args=(A.SKEL_FOLD, "float"), env=[F32, F32], out_rank=0, get=rd(0) + " * " + rd(1), combine="x + y", seed="0.0f"),
            "histogram": dict(args=(A.SKEL_PERMUTE, "Int32"), env=[I32], out_rank=1, get="1", combine="x + y", permutation=rd(0), combine_hint=A.COMBINE_ADD),
            "gaussian3x3": dict(args=(A.SKEL_STENCIL, "float"), out_rank=2, taps=[(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)], boundary="clamp",
                                stencil_fn=A.linear_stencil_fn([1, 2, 1, 2, 4, 2, 1, 2, 1], 16)),
            "smvm": dict(args=(A.SKEL_FOLDSEG, "float"), env=[F32, I32, F32], get=rd(0) + " * arrIn2_0[" + rd(1) + "]", combine="x + y", seed="0.0f"),
        }
        for name, kw in kinds.items():
            _, cold = build(name, 0, **dict(kw))                  # generated, compiled by hiprtc, loaded
            A.check(L.acc_cache_clear(0))                         # forget what memory holds, keep the files
            _, disk = build(name, 0, **dict(kw))
            _, ram = build(name, 0, **dict(kw))
            st[name] = {"cold_compile_ms": round(cold, 1), "disk_cache_load_ms": round(disk, 2), "ram_hit_us": round(ram * 1e3, 1)}
            log("  %-14s cold %8.1f ms   from the disk cache %6.2f ms   from memory %7.1f us" % (name, cold, disk, ram * 1e3))
        # the SMVM program's two kernels (the scan that makes the offsets, the segmented fold): compiled one after the
        # other, as acc_skel_create does, and side by side on the worker pool, as the front end's `run` has them
        t0 = time.perf_counter()
        build("pair", 1, **dict(kinds["scanl"]))
        build("pair", 1, **dict(kinds["smvm"]))
        serial = (time.perf_counter() - t0) * 1e3
        t0 = time.perf_counter()
        a_, _ = build("pair", 2, wait=False, **dict(kinds["scanl"]))
        b_, _ = build("pair", 2, wait=False, **dict(kinds["smvm"]))
        submitted = (time.perf_counter() - t0) * 1e3
        a_.wait()
        b_.wait()
        together = (time.perf_counter() - t0) * 1e3
        st["two_kernels"] = {"one_after_the_other_ms": round(serial, 1), "side_by_side_ms": round(together, 1),
                             "returned_to_the_caller_after_ms": round(submitted, 2), "compile_threads": int(L.acc_compile_threads())}
        log("  scanl + foldSeg: one after the other %.1f ms, side by side %.1f ms (the caller had both handles after %.2f ms)" % (serial, together, submitted))
        sk["startup"] = st

    if want("hostcost"):
        log("host time of a driver call (enqueue only) and small arrays ...")
        hc = {}
        small = 1024
        xs_ = ctx.array(np.arange(small, dtype=np.int32) % 7)
        o1, o2, tot = ctx.empty(small + 1, np.int32), ctx.empty(256, np.int32), ctx.empty((), np.int32)
        zero = ctx.array(np.zeros(256, np.int32))
        e1 = envs(xs_)
        m_ = ctx.skeleton(A.SKEL_MAP, "Int32", env=[I32], out_rank=1, get="arrIn0_0[ix] + 1", wait=True)
        f_ = ctx.skeleton(A.SKEL_FOLD, "Int32", env=[I32], out_rank=0, get="arrIn0_0[ix]", combine="x + y", seed="0", wait=True)
        s_ = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get="arrIn0_0[ix]", combine="x + y", seed="0", wait=True)
        p_ = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32], out_rank=1, get="1", combine="x + y", permutation="arrIn0_0[ix]", combine_hint=A.COMBINE_ADD, wait=True)
        od1, od1s, od2, zd, td = o1.desc(shape=(small,)), o1.desc(), o2.desc(), zero.desc(), tot.desc()
        sh1 = (C.c_int64 * 1)(small)
        calls = {
            "map": lambda: L.acc_exec_map(m_.handle, e1, C.byref(od1), stream),
            "fold": lambda: L.acc_exec_fold(f_.handle, e1, 1, sh1, C.byref(td), stream),
            "scan": lambda: L.acc_exec_scan(s_.handle, e1, small, C.byref(od1s), None, stream),
            "permute": lambda: L.acc_exec_permute(p_.handle, e1, small, C.byref(zd), C.byref(od2), stream),
        }
        empty_call = lambda: L.acc_launch_grid(1, 1, 1, 1)          # what a call through ctypes costs by itself
        reps = 3000
        t0 = time.perf_counter()
        for _ in range(reps):
            empty_call()
        ffi_us = (time.perf_counter() - t0) * 1e6 / reps
        for name, call in calls.items():
            for _ in range(200):
                call()
            ctx.sync()
            # host time: bursts short enough for the queue to take without the device having to catch up
            host_us = None
            for _ in range(12):
                t0 = time.perf_counter()
                for _ in range(128):
                    call()
                dt = (time.perf_counter() - t0) * 1e6 / 128
                host_us = dt if host_us is None else min(host_us, dt)
                ctx.sync()
            t0 = time.perf_counter()
            for _ in range(reps):
                call()
            ctx.sync()
            total_us = (time.perf_counter() - t0) * 1e6 / reps
            hc[name] = {"host_us_per_call": round(host_us, 2), "of_which_the_python_binding_us": round(ffi_us, 2),
                        "us_per_call_until_the_device_is_done": round(total_us, 2), "elements": small}
            log("  %-8s %6.2f us of host time a call (%.2f of them the ctypes call itself); %6.2f us a call with the device's work" % (name, host_us, ffi_us, total_us))
        # small arrays: device time a call, back to back
        rows = {}
        for lg in (10, 12, 14, 16, 18):
            nn = 1 << lg
            xa, oa = ctx.array(np.arange(nn, dtype=np.int32) % 7), ctx.empty(nn + 1, np.int32)
            ea, oda, odas = envs(xa), oa.desc(shape=(nn,)), oa.desc()
            sha = (C.c_int64 * 1)(nn)
            per = {}
            for name, call in (("map", lambda: A.check(L.acc_exec_map(m_.handle, ea, C.byref(oda), stream))),
                               ("fold", lambda: A.check(L.acc_exec_fold(f_.handle, ea, 1, sha, C.byref(td), stream))),
                               ("scan", lambda: A.check(L.acc_exec_scan(s_.handle, ea, nn, C.byref(odas), None, stream))),
                               ("permute", lambda: A.check(L.acc_exec_permute(p_.handle, ea, nn, C.byref(zd), C.byref(od2), stream)))):
                w_, e_ = T.run([call])
                per[name] = round(e_ * 1e3, 2)
            rows["2^%d" % lg] = per
            log("  n = 2^%-2d  us a call on the device, back to back: %s" % (lg, "  ".join("%s %.2f" % kv for kv in per.items())))
        hc["small_arrays_us_per_call"] = rows
        sk["host_cost"] = hc

    # ---------------------------------------------------------------- the same three computations built by the front end
    # (dot, scanl and SMVM written as array programs: what `run1` of the front end generates, compiles and launches
    # for them, timed kernel by kernel (acc_trace_start / acc_trace_stop: an event before and behind every launch),
    # beside the hand-written fragments above.  Host time per call is Python's and is not in these figures; a launch
    # onto an idle device carries a few microseconds of dispatch latency that back-to-back launches do not show.)
    if want("frontend"):
        log("front end: dotp, scanl and smvm as array programs ...")
        import accelerate_hip as acc
        fcx = acc.Context(0)
        fcx.N_STREAMS = 1                           # one stream: consecutive calls must not share the device, or each looks slower
        add = lambda a, b: a + b                    # noqa: E731
        K = max(4, min(args.steps, 20))

        def front(build, sets):
            acc_r = acc.compute(build(0), fcx)      # builds the skeletons, uploads the operands of set 0
            for i in range(1, sets):
                acc_r = acc.compute(build(i), fcx)
            fcx.ctx.sync()
            fcx.ctx.trace_start()                   # an event before and behind every launch the drivers make
            for k in range(K):
                acc_r = acc.compute(build(k % sets), fcx)
            launches, ms = fcx.ctx.trace_stop()
            return acc_r, round(ms * 1e3 / K, 3), launches // K

        fe = {}
        nd = 1 << 24
        x, y = wl.dot_inputs(nd)
        Sd = 4 * S
        xs, ys_ = [acc.use(x.copy(), fcx) for _ in range(Sd)], [acc.use(y.copy(), fcx) for _ in range(Sd)]
        r, us, nk = front(lambda i: acc.fold(add, 0.0, acc.zipWith(lambda a, b: a * b, xs[i], ys_[i]), context=fcx), Sd)
        fe["dot"] = {"gpu_us_per_call": us, "kernels_per_call": nk, "direct_avg_launch_us": sk.get("dot", {}).get("avg_launch_us"),
                     "direct_one_by_one_us": sk.get("dot", {}).get("one_by_one_us"),
                     "result": float(acc.run(r, fcx))}
        log("  front end dotp                 %9.3f us/call on the device, %d kernel(s); the hand-written fragment one by one: %s" % (us, nk, fe["dot"]["direct_one_by_one_us"]))
        del xs, ys_, r
        xsc = wl.scan_input(n)
        xs = [acc.use(xsc.copy(), fcx) for _ in range(S)]
        r, us, nk = front(lambda i: acc.scanl(add, 0, xs[i], context=fcx), S)
        got = acc.run(r, fcx)
        assert int(got[-1]) == int(xsc.sum(dtype=np.int64)), "front end scanl mismatch"
        fe["scanl"] = {"gpu_us_per_call": us, "kernels_per_call": nk, "direct_avg_launch_us": sk.get("scanl", {}).get("avg_launch_us"),
                       "direct_one_by_one_us": sk.get("scanl", {}).get("one_by_one_us")}
        log("  front end scanl                %9.3f us/call on the device, %d kernel(s); the hand-written fragment one by one: %s" % (us, nk, fe["scanl"]["direct_one_by_one_us"]))
        # `run1` as a user calls it (CUDA.hs:318-333): a host array in, a host array out, every call -- upload through
        # the memory table, the kernel, the result collected.  A new host array each time (one the table has seen is
        # not uploaded again, Array/Prim.hs:177-192); the kernels are built by the first call.
        del xs, r, got
        scan1 = acc.run1(lambda a: acc.scanl(add, 0, a, context=fcx), fcx)
        best = None
        for rep_ in range(4):
            fresh = xsc.copy()
            t0 = time.perf_counter()
            res1 = scan1(fresh)
            dt = time.perf_counter() - t0
            if rep_ and (best is None or dt < best):
                best = dt
            assert int(res1[-1]) == int(xsc.sum(dtype=np.int64))
            del res1, fresh
        fe["scanl"]["run1_ms"] = round(best * 1e3, 3)
        fe["scanl"]["run1_GB_per_s_over_the_link"] = round((2 * n * 4 + 4) / best / 1e9, 2)
        log("  front end run1 scanl           %9.3f ms a call, host array to host array (%.1f GB/s over the link)" % (best * 1e3, (2 * n * 4 + 4) / best / 1e9))
        del xsc
        vals, cols, offs, lens, xv = wl.smvm_inputs()
        vs, cs = [acc.use(vals.copy(), fcx) for _ in range(S)], [acc.use(cols.copy(), fcx) for _ in range(S)]
        vecs, ls = [acc.use(xv.copy(), fcx) for _ in range(S)], [acc.use(lens.copy(), fcx) for _ in range(S)]

        def smvm_prog(i):
            v = vecs[i]
            return acc.foldSeg(add, 0.0, acc.zipWith(lambda c, a: a * v[c], cs[i], vs[i]), ls[i], context=fcx)
        r, us, nk = front(smvm_prog, S)
        fe["smvm"] = {"gpu_us_per_call": us, "kernels_per_call": nk, "direct_avg_launch_us": sk.get("smvm", {}).get("avg_launch_us"),
                      "direct_one_by_one_us": sk.get("smvm", {}).get("one_by_one_us"),
                      "note": "per call: scanl of the 2^20 segment lengths into offsets, then foldSeg (the direct figure is foldSeg alone)"}
        log("  front end smvm                 %9.3f us/call on the device, %d kernel(s): offsets scan + foldSeg; the hand-written foldSeg one by one: %s" % (us, nk, fe["smvm"]["direct_one_by_one_us"]))
        del vs, cs, vecs, ls, r
        sk["front_end"] = fe
        acc.destroy(fcx)

    # ---------------------------------------------------------------- not a configuration: fold along rows of 64
    # (only when named: the rows of a rank-2 array are segments whose starts lie a multiple of 32 elements apart, the
    # case the padding of the staged chunk in LDS is there for; ACC_HIP_TUNE=foldseg.pad=0 runs it without)
    if "foldrows64" in only:
        log("fold (+) along the rows of a 2^20 x 64 Float32 array ...")
        rows, width = 1 << 20, 64
        m = wl.dot_inputs(rows * width)[0].reshape(rows, width)
        dms = [ctx.array(m) for _ in range(S)]
        env_s = [envs(d) for d in dms]
        rs = [ctx.empty(rows, np.float32) for _ in range(S)]
        frow = ctx.skeleton(A.SKEL_FOLD, "float", env=[(2, "float")], out_rank=1, get=rd(0), combine="x + y", seed="0.0f")
        rds = [r.desc() for r in rs]
        sh2 = (C.c_int64 * 2)(rows, width)

        def step(i):
            return lambda: A.check(L.acc_exec_fold(frow.handle, env_s[i], 2, sh2, C.byref(rds[i]), stream))
        w, e = T.run([step(i) for i in range(S)])
        want_rows = m[:, 0].copy()
        for k in range(1, width):
            want_rows += m[:, k]                      # left to right in Float32, as the kernel folds a row
        assert np.array_equal(rs[S - 1].get(), want_rows), "row sums mismatch"
        sk["foldrows64"] = result("fold (+) rows of 64 Float32", w, e, 1, rows * width * 4 + rows * 4, rows * width)
        del dms, env_s, rs, m

    # ---------------------------------------------------------------- not a configuration: other shapes and sizes
    # (only when named: small scans, which take small tiles; stencils on volumes of few strips, on arrays narrower than
    # a strip and over 8-byte elements; a transpose in runs and in tiles)
    if "shapes" in only:
        log("other shapes and sizes (us per launch, every launch on the same buffers) ...")
        shapes = {}

        def one(name, fn, nbytes):
            w, e = T.run([fn])
            shapes[name] = {"avg_launch_us": round(e * 1e3, 2), "GB_per_s": round(nbytes / (e * 1e-3) / 1e9, 1)}
            log("  %-44s %9.2f us/launch  %8.1f GB/s" % (name, e * 1e3, nbytes / (e * 1e-3) / 1e9))

        scan_s = ctx.skeleton(A.SKEL_SCANL, "Int32", env=[I32], get=rd(0), combine="x + y", seed="0")
        for n in (1 << 10, 49155, 1 << 18, 1 << 21, (3 << 20) + 3, 1 << 22, 1 << 24):
            x, o = ctx.array(np.ones(n, np.int32)), ctx.empty(n + 1, np.int32)
            xe, od = envs(x), o.desc()
            one("scanl (+) Int32 n = %d" % n, lambda: A.check(L.acc_exec_scan(scan_s.handle, xe, n, C.byref(od), None, stream)), 8 * n)
            del x, o
        seven = [(0, 0, 0), (-1, 0, 0), (1, 0, 0), (0, -1, 0), (0, 1, 0), (0, 0, -1), (0, 0, 1)]
        nine = [(dy, dx) for dy in (-1, 0, 1) for dx in (-1, 0, 1)]
        for ctype, dt in (("float", np.float32), ("double", np.float64)):
            lap3 = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=3, taps=seven, boundary="clamp", stencil_fn="t1 + t2 + t3 + t4 + t5 + t6 - 6 * t0")
            box2 = ctx.skeleton(A.SKEL_STENCIL, ctype, out_rank=2, taps=nine, boundary="clamp", stencil_fn=" + ".join("t%d" % k for k in range(9)))
            vols = ((512, 512, 512), (384, 384, 384), (300, 300, 300), (256, 256, 256), (150, 150, 150), (128, 128, 256), (100, 400, 419), (1024, 128, 128), (4096, 64, 64), (1 << 22, 2, 2)) if ctype == "float" else ((256, 512, 512),)
            for shape in vols:
                a, o = ctx.array(np.ones(shape, dt)), ctx.empty(shape, dt)
                ad, od = a.desc(), o.desc()
                one("stencil 7-point %s %d x %d x %d" % ((ctype,) + shape), lambda: A.check(L.acc_exec_stencil(lap3.handle, None, C.byref(ad), C.byref(od), stream)),
                    2 * int(np.prod(shape)) * np.dtype(dt).itemsize)
                del a, o
            imgs = ((1 << 17, 128), (1 << 18, 64), (55924, 300), (1 << 24, 3)) if ctype == "float" else ((8192, 8192),)
            for shape in imgs:
                a, o = ctx.array(np.ones(shape, dt)), ctx.empty(shape, dt)
                ad, od = a.desc(), o.desc()
                one("stencil 3x3 %s %d x %d" % ((ctype,) + shape), lambda: A.check(L.acc_exec_stencil(box2.handle, None, C.byref(ad), C.byref(od), stream)),
                    2 * int(np.prod(shape)) * np.dtype(dt).itemsize)
                del a, o
        side = 8192
        src, dst = ctx.array(wl.stencil_image(side, side)), ctx.empty((side, side), np.float32)
        se, dd = envs(src), dst.desc()
        for name, flags in (("in runs", 0), ("in tiles (ACC_FLAG_TILED)", A.FLAG_TILED)):
            tr = ctx.skeleton(A.SKEL_MAP, "float", env=[(2, "float")], out_rank=2, flags=flags, get="arrIn0_0[(ix % shOut_0) * shIn0_0 + (ix / shOut_0)]")
            one("transpose 8192 x 8192 Float32 " + name, lambda: A.check(L.acc_exec_map(tr.handle, se, C.byref(dd), stream)), 8 * side * side)
        assert np.array_equal(dst.get(), wl.stencil_image(side, side).T), "transpose mismatch"
        del src, dst
        # (a result of two rows or two columns: most of every tile would lie outside it, so the tiled instance goes in runs)
        for shape in ((1 << 23, 2), (2, 1 << 23)):
            thin = np.arange(shape[0] * shape[1], dtype=np.float32).reshape(shape)
            src, dst = ctx.array(thin), ctx.empty((shape[1], shape[0]), np.float32)
            se, dd = envs(src), dst.desc()
            one("transpose %d x %d Float32 (ACC_FLAG_TILED)" % shape, lambda: A.check(L.acc_exec_map(tr.handle, se, C.byref(dd), stream)), 8 * thin.size)
            assert np.array_equal(dst.get(), thin.T), "transpose mismatch"
            del src, dst
        # segmented sums whose lengths are very unequal: a million segments of 8 elements on average, one of which holds
        # half of the source (the rows of a power-law graph), folded by its workgroup alone (`foldseg.giants=0`) and handed
        # over to a second launch (`=1`; as the knobs stand an instance goes from the one to the other by itself, once
        # it has looked at its segment lengths and the other variant is compiled); the same elements all in segments of 8
        nseg, big = 1 << 20, 1 << 23
        for name, giant, knobs in (("every segment short", 0, ""), ("one segment of 2^23 elements among them, foldseg.giants=0", big, "foldseg.giants=0"),
                                   ("one segment of 2^23 elements among them, foldseg.giants=1", big, "foldseg.giants=1")):
            with A.tuning(knobs, ctx):
                seg_s = ctx.skeleton(A.SKEL_FOLDSEG, "float", env=[F32], get=rd(0), combine="x + y", seed="0.0f")
            rng_l = np.random.default_rng(5)
            lens = rng_l.poisson(8, nseg).astype(np.int64)
            if giant:
                lens[nseg // 3] = giant
            else:
                lens = np.concatenate([lens, rng_l.poisson(8, big // 8).astype(np.int64)])
            offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            nel = int(offs[-1])
            xv_ = ctx.array(np.ones(nel, np.float32))
            do_, out_ = ctx.array(offs), ctx.empty(lens.size, np.float32)
            xe, dd_, od_ = envs(xv_), do_.desc(), out_.desc()
            one("foldSeg (+) Float32, %d segments, %s" % (lens.size, name),
                lambda: A.check(L.acc_exec_foldseg(seg_s.handle, xe, nel, C.byref(dd_), C.byref(od_), stream)), 4 * nel + 8 * lens.size)
            assert np.array_equal(out_.get(), lens.astype(np.float32)), "segmented sums mismatch"
            del xv_, do_, out_
            seg_s.destroy()
        # sums down the columns of a matrix, written as the fold of its transpose: the rows that the fold sees lie
        # across memory -- teams of lanes along them (no flag) against a lane a row (ACC_FLAG_TILED)
        for shape in ((4096, 4096), (1 << 16, 256)):
            mat = np.ones(shape, np.float32)
            src, dst = ctx.array(mat), ctx.empty(shape[1], np.float32)
            se, dd = envs(src), dst.desc()
            ext = (C.c_int64 * 2)(shape[1], shape[0])
            # (the index as a code generator writes it: the extents as literals; over the kernel's names for the row
            # and the place within it where a lane takes a row)
            for name, flags, text in (("teams of lanes", 0, "arrIn0_0[(ix %% %dLL) * %dLL + ix / %dLL]" % (shape[0], shape[1], shape[0])),
                                      ("a lane a row (ACC_FLAG_TILED)", A.FLAG_TILED, "arrIn0_0[acc_col * %dLL + acc_row]" % shape[1])):
                cs = ctx.skeleton(A.SKEL_FOLD, "float", env=[(2, "float")], out_rank=1, flags=flags, combine="x + y", seed="0.0f", get=text)
                one("fold (+) of the transpose of %d x %d Float32, %s" % (shape + (name,)),
                    lambda: A.check(L.acc_exec_fold(cs.handle, se, 2, ext, C.byref(dd), stream)), 4 * mat.size)
                assert np.array_equal(dst.get(), mat.sum(axis=0)), "column sums mismatch"
                cs.destroy()
            del src, dst
        # `permute const`, every target written once: the scatter of a stream compaction (half of the sources kept, in
        # order) and of a stable sorting pass by a 4-bit digit; stores (as the knobs stand) against a read and a
        # compare-and-swap an element (`permute.replace=0`)
        nper = 1 << 24
        rng_p = np.random.default_rng(9)
        vals_p = rng_p.integers(0, 1 << 30, nper).astype(np.int32)
        keep_p = rng_p.random(nper) < 0.5
        places_p = np.where(keep_p, np.cumsum(keep_p) - keep_p, -1).astype(np.int32)
        order_p = np.argsort(vals_p & 15, kind="stable")
        dest_p = np.empty(nper, np.int32)
        dest_p[order_p] = np.arange(nper, dtype=np.int32)
        dv_p = ctx.array(vals_p)
        for name, tgt, nt in (("a compaction, half of the sources kept", places_p, int(keep_p.sum())), ("a sorting pass by a 4-bit digit", dest_p, nper)):
            dk_p, dfl_p, out_p = ctx.array(tgt), ctx.array(np.zeros(nt, np.int32)), ctx.empty(nt, np.int32)
            pe, pd, po = envs(dk_p, dv_p), dfl_p.desc(), out_p.desc()
            want_p = np.zeros(nt, np.int32)
            want_p[tgt[tgt >= 0]] = vals_p[tgt >= 0]
            for knobs in ("", "permute.replace=0"):
                with A.tuning(knobs, ctx):
                    pc = ctx.skeleton(A.SKEL_PERMUTE, "Int32", env=[I32, I32], out_rank=1, get="arrIn1_0[ix]", combine="x", permutation="(Int64)arrIn0_0[ix]")
                one("permute const Int32, 2^24 sources, %s%s" % (name, ", " + knobs if knobs else ""),
                    lambda: A.check(L.acc_exec_permute(pc.handle, pe, nper, C.byref(pd), C.byref(po), stream)), 8 * nper + 8 * nt)
                assert np.array_equal(out_p.get(), want_p), "permute const mismatch"
                pc.destroy()
            del dk_p, dfl_p, out_p
        del dv_p
        sk["shapes"] = shapes

    if headline is None:     # --only without scan: report whatever ran first
        timed = sorted(k for k in sk if "ms_per_step" in sk[k])
        if not timed:
            print(json.dumps({"skeletons": sk}))
            ctx.close()
            return
        k0 = timed[0]
        headline = dict(sk[k0], wall_ms=sk[k0]["ms_per_step"], event_ms=sk[k0]["event_ms_per_step"])
        workload = k0
    else:
        workload = "configs[1]: scanl (+) 0 over 2^26 Int32, values uniform in [0,16)"

    line = {
        "metric": "effective GB/s of the scan skeleton (algorithmic bytes / time); per-skeleton figures under 'skeletons'",
        "value": headline["GB_per_s"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": headline["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int32", "data": "synthetic (seeded SplitMix64, resident in HBM before the timed region)",
        "config": {"workload": workload, "elements": n, "buffer_sets": S,
                   "timing": "kernel launches back to back on one stream, inputs device-resident, consecutive launches on different buffer sets; %d ms of untimed launches before the warm-up steps of every configuration that finds the device idle" % int(Timer.DEVICE_WARMUP_MS)},
        "roofline": {"bound": "hbm", "achieved": headline["GB_per_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(headline["GB_per_s"] / HBM_PEAK_GBS, 4),
                     "traffic": headline.get("hbm_traffic_bytes"), "traffic_source": headline.get("hbm_traffic_source"),
                     "traffic_kernel_sources_sha256": profile_hash(os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.txt")),
                     "kernel_sources_sha256": kernel_sources_hash(), "stale": headline.get("hbm_traffic_stale"),
                     "kernel": "scanl", "avg_launch_us": headline["avg_launch_us"],
                     "algorithmic_bytes_per_launch": headline["algorithmic_bytes_per_launch"]},
        "cpu_baseline": cpu,
        "skeletons": sk,
    }
    print(json.dumps(line))
    ctx.close()


if __name__ == "__main__":
    main()
