#!/usr/bin/env python3
"""
Benchmark of Heat's k-means Lloyd path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config all|c1..c5] [--no-cpu-baseline]

Prints ONE JSON line.  Without --config it measures the headline workload (c3: N = 10M, D = 32, K = 256) in
full and then the other four workloads' figures, which the same line carries under `configs`.

value      what the reference's own benchmark reports (benchmarks/2020/kmeans/heat-cpu.py:22-25): the wall time of
           ht.cluster.KMeans(n_clusters=K, init=C0, max_iter=T, tol=0).fit(x) through the public estimator, from
           the workload's seeded init with its own iteration count T, as N * n_iter_ / wall time.  Inputs are
           resident in HBM; the clock runs between two synchronisations around the call and so covers the copy of
           the init, every buffer the fit allocates, the T iterations with the host's look at every shift, and
           the (N, 1) int64 labels.  `fit` holds the details: fit_ms (median of max(5, K / T) fits that follow one
           warm fit), first_fit_ms (the first fit on the resident data, before anything else ran), n_iter, and
           `checked`: after the last timed fit, every row has a label in [0, K) and the two-pass means of those
           labels reproduce cluster_centers_ to 1e-6.  ms_per_step = fit_ms / n_iter.
steady_state  the same step in a long loop (heat_amd.cluster._lloyd.LloydLoop: one hkm_lloyd_step_f32 per iteration,
           the host reads every 4-byte shift, the next step is enqueued while it does), W warm-up steps (at least
           30 run before timing: a kernel launched on an idle device runs up to 30 % longer during the first
           ~25 ms of load), then five timed regions of K steps; the median region is reported.
roofline   the dominant kernel -- the fused distance+argmin kernel, or the one-sweep kernel that also forms
           the per-cluster sums -- timed ALONE: the library records an event pair on the launch stream
           right around that kernel's launch (hkm_profile_enable) during one more pass of K steps; kernel_ms is
           the mean over those launches, achieved = algorithmic flops 2*N*K*D (MFMA-bound shapes) or bytes
           N*(4D+4) (HBM-bound shapes) per launch / kernel_ms.
           traffic (HBM bytes per launch, rocprofv3 FETCH_SIZE / WRITE_SIZE) is read from
           profiles/traffic.json and only reported while the library sources still hash to what they
           were when it was measured (traffic_source says which); traffic_frac = traffic / kernel_ms / 8 TB/s,
           the share of the HBM peak the kernel really moves (for the narrow one-sweep step, which stores no
           labels, that is less than `frac`, which prices the algorithmic bytes).
           step_ms_events is the whole step (all its launches, no host read) between two events.
           sclk_mhz_under_load is the shader clock the driver reports while that step runs back to
           back (peak assumes 2400 MHz; chips differ in what they hold under the matrix-core kernels),
           mfma_alone_tflops_this_chip what a chain of nothing but fp32 matrix instructions reaches on
           this chip right after (the probe of --probe)
cpu_baseline  the CPU restatement of the reference's op sequence (oracle/, torch CPU, all host
           threads) on a bounded row sample of the headline workload
configs    c1, c2, c4, c5 (only without --config): value (fit-based; c2: points/s of the assignment), fit_ms,
           first_fit_ms, n_iter, the steady-state step, kernel_ms, frac, traffic, traffic_frac, checked

--shape N D K times the same loop on K equal blobs of any shape (the lines of profiles/bench_other_shapes.jsonl);
such a line has no CPU baseline and no traffic figure and is no headline number.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# The sources whose code runs in each clustering workload: dispatch and shared headers, then the file of the
# workload's kernels (the narrow one-sweep kernel for c1 and c5, the matrix-core kernels for c2-c4, with
# the two-pass update c4 runs and c3 falls back to).  A counter reading is tied to these.
_SHARED_SOURCES = ("hkm_api.hip", "hkm_common.h", "hkm_mfma_util.h")
_MFMA_SOURCES = _SHARED_SOURCES + ("hkm_assign_mfma.hip", "hkm_update.hip", "hkm_update_sorted.hip")
WORKLOAD_SOURCES = {"c1": _SHARED_SOURCES + ("hkm_lloyd_small.hip",), "c5": _SHARED_SOURCES + ("hkm_lloyd_small.hip",),
                    "c2": _SHARED_SOURCES + ("hkm_assign_mfma.hip",), "c3": _MFMA_SOURCES, "c4": _MFMA_SOURCES}


def workload_sources_sha1(config: str) -> str:
    """Hash of the HIP sources behind one workload's kernels: ties a committed counter reading to the code."""
    import hashlib

    h = hashlib.sha1()
    for name in WORKLOAD_SOURCES[config]:
        with open(os.path.join(ROOT, "heat_amd", "csrc", name), "rb") as fh:
            h.update(name.encode() + b"\0" + fh.read())
    return h.hexdigest()[:12]


PEAK_HBM_GBS = 8000.0
PEAK_FP32_MFMA_TFLOPS = 157.3
# configs that are bound by the fp32 matrix pipe; the others stream X from HBM
MFMA_BOUND = {"c2", "c3", "c4"}
# rows of the CPU baseline's sample = N / divisor: about 5-20 s of host work per workload
CPU_SAMPLE_DIV = {"c1": 1, "c2": 1, "c3": 16, "c4": 128, "c5": 8}


def run_probe() -> int:
    """bench.py --probe: the hardware figures the kernels are designed around, measured with the library's
    microbenchmark kernels (hkm_probe_mfma_f32, hkm_probe_stream) and device events.  One JSON line."""
    import ctypes

    import torch

    from heat_amd.utils import benchhooks

    lib = benchhooks.bench()
    check = benchhooks.check_probe
    dev = torch.device("cuda:0")
    P = ctypes.c_void_p

    def timed(fn, reps):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    stream = P(torch.cuda.current_stream().cuda_stream)
    grid, iters = 1024, 2000
    out = torch.empty((grid * 256,), dtype=torch.float32, device=dev)
    flops = grid * 4 * iters * 16 * 4096.0
    res = {"probe": "mfma+stream", "mfma_f32_32x32x2": {}, "stream": {}}
    # warm the clocks
    timed(lambda: check(lib.hkm_probe_mfma_f32(0, 0, iters, grid, P(out.data_ptr()), stream)), 20)
    base_ms = timed(lambda: check(lib.hkm_probe_mfma_f32(0, 0, iters, grid, P(out.data_ptr()), stream)), 10)
    base_tf = flops / (base_ms * 1e-3) / 1e12
    res["mfma_f32_32x32x2"]["alone_tflops"] = round(base_tf, 1)
    res["mfma_f32_32x32x2"]["alone_frac_of_157.3"] = round(base_tf / 157.3, 3)
    names = {1: "v_fma_f32", 2: "v_cndmask_b32", 3: "v_min3_f32", 4: "s_add_u32", 5: "v_cmp_lt_f32", 6: "v_mov_b64"}
    for op, name in names.items():
        ms = timed(lambda: check(lib.hkm_probe_mfma_f32(op, 8, iters, grid, P(out.data_ptr()), stream)), 10)
        # cycles one matrix instruction's slot grows by per interleaved instruction (64 cycles = the matrix instruction alone)
        res["mfma_f32_32x32x2"][f"cycles_per_{name}"] = round(64.0 * (ms / base_ms - 1.0) / 8.0, 2)
    nbytes = 2_400_000_000
    a = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    b = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    a.zero_()
    sink = torch.zeros((1,), dtype=torch.float32, device=dev)
    for mode, name, moved in ((0, "copy", 2 * nbytes), (1, "read", nbytes), (2, "read_nontemporal", nbytes), (3, "fill", nbytes)):
        ms = timed(lambda: check(lib.hkm_probe_stream(P(a.data_ptr()), P(b.data_ptr()), nbytes, mode,
                                                              P(sink.data_ptr()), stream)), 20)
        res["stream"][f"{name}_TBps"] = round(moved / (ms * 1e-3) / 1e12, 2)
    res["stream"]["bytes"] = nbytes
    print(json.dumps(res))
    return 0


def bench_kmedians(args, w, x, t_gen) -> int:
    """One KMedians iteration = fused Manhattan distance+argmin, per-cluster medians, centroid shift
    and its 4-byte read, as KMedians.fit issues them.  The dominant kernel is the assignment; it is
    bound by the fp32 vector ALU (2 lane-operations per point, centroid and feature; peak 256 CUs x 64
    lanes x 2.4 GHz = 39.3 T lane-op/s, i.e. the 78.6 TFLOP/s of unpacked vector FMA)."""
    import torch

    from heat_amd import _native

    if w.init is None:
        print("--estimator kmedians needs a clustering workload (not c2)", file=sys.stderr)
        return 2
    dev = x.device
    n, d = x.shape
    k = w.k
    ws = _native.Workspace(dev)
    lab = torch.empty((n,), dtype=torch.int32, device=dev)
    shift = torch.zeros((), dtype=torch.float32, device=dev)
    state = {"c": w.init.to(dev).clone()}
    fb = torch.zeros((k,), dtype=torch.int64, device=dev)

    def step():
        _native.assign_l1(x, state["c"], lab, None)
        c_new = torch.empty_like(state["c"])
        _native.update_median(x, lab, c_new, ws, fallback_rows=fb, skip_zero_rows=True)
        _native.shift(state["c"], c_new, shift)
        state["c"] = c_new
        shift.item()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ev = []
    for _ in range(args.steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _native.assign_l1(x, state["c"], lab, None)
        e1.record()
        torch.cuda.synchronize()
        ev.append(e0.elapsed_time(e1))
    kern_ms = sum(ev) / len(ev)
    ops = 2.0 * n * k * d
    peak = 39.3216
    out = {
        "metric": "KMedians points*iter/s", "value": round(n * args.steps / elapsed, 1), "unit": "points*iter/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {t_gen:.1f} s, resident in HBM before timing)",
        "config": {"workload": w.name, "estimator": "KMedians", "N": n, "D": d, "K": k, "scale": args.scale},
        "roofline": {"bound": "valu", "achieved": round(ops / (kern_ms * 1e-3) / 1e12, 3), "peak": peak,
                     "unit": "Tlane-op/s", "frac": round(ops / (kern_ms * 1e-3) / 1e12 / peak, 4),
                     "kernel": "l1_argmin", "kernel_ms": round(kern_ms, 4), "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(out))
    return 0


def bench_init(args, w, x, t_gen) -> int:
    """The k-means|| initialiser (KMeans(init="probability_based"), heat/cluster/_kcluster.py:146-247) on
    the workload's data: a "step" is one complete initialisation -- the sampling rounds (one fused
    distance + minimum launch against the round's new candidates, a reduction, an ordered selection),
    the weights of the candidates and their k-means++ reclustering.  oversampling = 20 (with the
    reference's default of 2 fewer candidates than clusters come out for K = 256 and the reference
    restarts with 20 itself).  The rounds are bound by reading X once each: algorithmic bytes per step
    = (rounds + 2) * N * 4 D (initial cost, one read per round but the last, the final assignment)."""
    import warnings

    import torch

    import heat_amd as ht

    if w.init is None:
        print("--estimator init needs a clustering workload (not c2)", file=sys.stderr)
        return 2
    n, d = x.shape
    k = w.k
    xd = ht.array(x, split=0)

    def step(seed):
        km = ht.cluster.KMeans(n_clusters=k, init="probability_based", random_state=seed)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            km._initialize_cluster_centers(xd, 20, 1)
        return km

    for i in range(min(args.warmup, 5)):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        km = step(100 + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    nrounds = int(km._init_rounds)  # int(ln(initial cost)) of the last seed
    alg = (nrounds + 2) * n * 4.0 * d
    ms = elapsed / args.steps * 1e3
    out = {
        "metric": "k-means|| initialisation points/s", "value": round(n * args.steps / elapsed, 1), "unit": "points/s",
        "n_gpus": 1, "steps": args.steps, "warmup": min(args.warmup, 5), "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {t_gen:.1f} s, resident in HBM before timing)",
        "config": {"workload": w.name, "estimator": "KMeans(init=probability_based)", "N": n, "D": d, "K": k,
                   "oversampling": 20, "rounds": nrounds, "scale": args.scale},
        "roofline": {"bound": "hbm", "achieved": round(alg / (ms * 1e-3) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                     "frac": round(alg / (ms * 1e-3) / 8e12, 4), "kernel": "whole initialisation (host-timed)",
                     "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(out))
    return 0


def bench_cdist(args, w, x, t_gen) -> int:
    """The public full-matrix ht.spatial.cdist(X, Y, quadratic_expansion=True) on rows of the c2 data:
    X = the first 32768 rows, Y = the next 32768 rows (D = 64), a 4.29 GB matrix of sqrt distances per
    step, written into one resident output buffer through the C ABI.  flops = 2 M N D."""
    import torch

    from heat_amd import _native

    if args.config != "c2":
        print("--estimator cdist runs on the c2 data", file=sys.stderr)
        return 2
    m = nn = min(32768, x.shape[0] // 2)
    d = x.shape[1]
    xa, ya = x[:m], x[m:m + nn]
    out = torch.empty((m, nn), dtype=torch.float32, device=x.device)

    def step():
        _native.pairwise(xa, ya, out, _native.METRIC_EUCLID_QE)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ev = []
    for _ in range(args.steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step()
        e1.record()
        torch.cuda.synchronize()
        ev.append(e0.elapsed_time(e1))
    kern_ms = sum(ev) / len(ev)
    flops = 2.0 * m * nn * d
    out_bytes = 4.0 * m * nn
    res = {
        "metric": "cdist GFLOP/s", "value": round(flops * args.steps / elapsed / 1e9, 1), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {t_gen:.1f} s, resident in HBM before timing)",
        "config": {"workload": f"cdist_full_m{m}_n{nn}_d{d}", "M": m, "N": nn, "D": d, "scale": args.scale},
        "roofline": {"bound": "mfma", "achieved": round(flops / (kern_ms * 1e-3) / 1e12, 3), "peak": 157.3,
                     "unit": "TFLOP/s", "frac": round(flops / (kern_ms * 1e-3) / 1e12 / 157.3, 4),
                     "hbm_frac": round(out_bytes / (kern_ms * 1e-3) / 8e12, 4),
                     "kernel": "cdist_mfma", "kernel_ms": round(kern_ms, 4), "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(res))
    return 0


def bench_knn(args, w, x, t_gen) -> int:
    """k nearest rows + label vote (KNeighborsClassifier.predict, k = 5) on rows of the c2 data: test rows =
    the first 32768 rows, training rows = the next 32768 (D = 64), 10 classes.  flops = 2 M N D (the
    products on the matrix cores); the 4.29 GB distance matrix is never formed."""
    import torch

    from heat_amd import _native

    if args.config != "c2":
        print("--estimator knn runs on the c2 data", file=sys.stderr)
        return 2
    m = nn = min(32768, x.shape[0] // 2)
    d = x.shape[1]
    k, ncls = 5, 10
    q, train = x[:m], x[m:m + nn]
    g = torch.Generator(device=x.device).manual_seed(w.seed)
    y = torch.zeros((nn, ncls), dtype=torch.float32, device=x.device)
    y.scatter_(1, torch.randint(0, ncls, (nn, 1), device=x.device, generator=g), 1.0)
    idx = torch.empty((m, k), dtype=torch.int64, device=x.device)
    cls = torch.empty((m,), dtype=torch.int64, device=x.device)
    ws = _native.Workspace(x.device)

    def step():
        _native.knn(q, train, k, idx, None, ws)
        _native.knn_vote(idx, y, cls)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ev = []
    for _ in range(args.steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step()
        e1.record()
        torch.cuda.synchronize()
        ev.append(e0.elapsed_time(e1))
    kern_ms = sum(ev) / len(ev)
    flops = 2.0 * m * nn * d
    res = {
        "metric": "kNN predict test rows/s", "value": round(m * args.steps / elapsed, 1), "unit": "rows/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {t_gen:.1f} s, resident in HBM before timing)",
        "config": {"workload": f"knn_predict_m{m}_n{nn}_d{d}_k{k}", "M": m, "N": nn, "D": d, "k": k,
                   "classes": ncls, "scale": args.scale},
        "roofline": {"bound": "mfma", "achieved": round(flops / (kern_ms * 1e-3) / 1e12, 3), "peak": 157.3,
                     "unit": "TFLOP/s", "frac": round(flops / (kern_ms * 1e-3) / 1e12 / 157.3, 4),
                     "kernel": "knn_mfma_lds + knn_merge + knn_vote (whole step)", "kernel_ms": round(kern_ms, 4),
                     "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(res))
    return 0


def bench_silhouette(args, w, x, t_gen) -> int:
    """ht.cluster.silhouette_samples on the first 100 000 rows of the c3 data (D = 32) with their labels
    from one assignment against the workload's K = 256 centroids: per-sample, per-cluster distance sums
    without the 40 GB distance matrix.  Work = 2 N^2 D vector operations (subtract, fused multiply-add)
    plus one square root per pair; peak 39.3 T lane-ops/s (256 CUs x 64 lanes x 2.4 GHz)."""
    import torch

    import heat_amd as ht
    from heat_amd import _native

    if args.config != "c3":
        print("--estimator silhouette runs on the c3 data", file=sys.stderr)
        return 2
    n = min(100000, x.shape[0])
    d = x.shape[1]
    xs = x[:n].contiguous()
    lab = torch.empty((n,), dtype=torch.int32, device=x.device)
    _native.assign(xs, w.init.to(x.device), lab, None, _native.Workspace(x.device))
    X, L = ht.array(xs, split=0), ht.array(lab.long(), split=0)

    def step():
        return ht.cluster.silhouette_samples(X, L)

    for _ in range(min(args.warmup, 3)):
        step()
    torch.cuda.synchronize()
    steps = min(args.steps, 10)
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops = 2.0 * n * n * d
    ms = elapsed / steps * 1e3
    res = {
        "metric": "silhouette samples/s", "value": round(n * steps / elapsed, 1), "unit": "samples/s",
        "n_gpus": 1, "steps": steps, "warmup": min(args.warmup, 3), "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {t_gen:.1f} s, resident in HBM before timing)",
        "config": {"workload": f"silhouette_n{n}_d{d}_k{w.k}", "N": n, "D": d, "K": w.k, "scale": args.scale,
                   "mean_coefficient": round(float(out.larray.mean()), 6)},
        "roofline": {"bound": "valu", "achieved": round(ops / (ms * 1e-3) / 1e12, 3), "peak": 39.3,
                     "unit": "T lane-ops/s", "frac": round(ops / (ms * 1e-3) / 1e12 / 39.3, 4),
                     "kernel": "silhouette_sums (whole call: sort of the labels, sums, coefficients)",
                     "kernel_ms": round(ms, 4), "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(res))
    return 0


def mfma_alone_tflops() -> float:
    """What this chip sustains on fp32 matrix instructions and nothing else (the chain of bench.py --probe,
    about 0.4 s of it, clocks already warm): the ceiling `frac` could reach here if the kernel issued
    nothing but matrix instructions.  Chips differ: some hold 2.4 GHz under it, some do not."""
    import ctypes

    import torch

    from heat_amd.utils import benchhooks

    lib = benchhooks.bench()
    check = benchhooks.check_probe
    grid, iters = 1024, 2000
    out = torch.empty((grid * 256,), dtype=torch.float32, device="cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    flops = grid * 4 * iters * 16 * 4096.0

    def run(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            check(lib.hkm_probe_mfma_f32(0, 0, iters, grid, ctypes.c_void_p(out.data_ptr()), stream))
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    run(40)
    return flops / (run(40) * 1e-3) / 1e12


def sclk_under_load(enqueue, seconds: float = 0.6):
    """Median of the current shader clock (MHz) as /sys/class/drm/card*/device/pp_dpm_sclk reports it while
    `enqueue` keeps the device busy; the first 0.2 s are left out (the clock ramps up)."""
    import glob

    import torch

    files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    if not files:
        return None
    vals = []
    t0 = time.perf_counter()
    try:
        while time.perf_counter() - t0 < seconds:
            enqueue()
            if time.perf_counter() - t0 < 0.2:
                continue
            with open(files[0]) as f:
                for line in f:
                    if "*" in line:
                        vals.append(int(line.split(":")[1].strip().split("Mhz")[0]))
    except (OSError, ValueError, IndexError):
        vals = []
    torch.cuda.synchronize()
    if not vals:
        return None
    return sorted(vals)[len(vals) // 2]


def _traffic(config: str, wname: str, scale: float, shape) -> tuple:
    """(HBM bytes per launch of the workload's dominant kernel from profiles/traffic.json or None, where from)."""
    tfile = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(tfile):
        return None, "none: profiles/traffic.json is missing"
    with open(tfile) as f:
        tj = json.load(f)
    if config not in WORKLOAD_SOURCES or shape:
        return None, "none: profiles/traffic.json holds the five named workloads only"
    if scale != 1.0:
        return None, "dropped: profiles/traffic.json holds the unscaled workloads only"
    sha = workload_sources_sha1(config)
    measured_on = (tj.get("sources_sha1") or {}).get(wname)
    if measured_on == sha:
        return tj.get(wname), f"profiles/traffic.json, measured on this workload's kernel sources sha1 {sha} (= this build)"
    return None, f"dropped: profiles/traffic.json was measured on kernel sources sha1 {measured_on}, this build is {sha}"


def measure(args, config: str, headline: bool) -> dict:
    """One workload, measured two ways.

    fit     ht.cluster.KMeans(n_clusters=K, init=C0, max_iter=T, tol=0.0).fit(x) through the public estimator, from
            the workload's own seeded init with its own T, wall clock between two synchronisations: what the
            reference's own benchmark times (benchmarks/2020/kmeans/heat-cpu.py:22-25 around
            heat/cluster/kmeans.py:105-148).  first_fit_ms is the first fit on the resident data, before anything
            else ran on it; fit_ms the median of the timed fits that follow the warm-up.  After the last timed fit
            its own result is checked: every row has a label, and the two-pass means of the returned labels
            reproduce cluster_centers_ to 1e-6.  (c2 has no fit: its call is one assignment, checked against
            float64 distances on a sample of rows.)
    steady  the Lloyd step in a long loop, as before: median of `regions` timed regions of `steps` steps.
    The headline workload gets the full line (clock, probe, CPU baseline); the others the figures only."""
    import torch

    import heat_amd as ht
    from heat_amd import _native
    from heat_amd.cluster._lloyd import LloydLoop
    from heat_amd.utils import benchhooks, synthetic

    dev = torch.device("cuda:0")
    t_gen = time.perf_counter()
    if args.shape:
        config = "shape"
        w = synthetic.shape(*args.shape)
    else:
        w = synthetic.CONFIGS[config](args.scale)
    t_gen = time.perf_counter() - t_gen
    n, d = w.x.shape
    k = w.k
    x = w.x.to(dev)
    torch.cuda.synchronize()
    is_assign = config == "c2"
    kernel = _native.assign_kernel_name(n, d, k) if is_assign else _native.lloyd_kernel_name(n, d, k)
    kernel = kernel.replace("+update", "")
    ws = _native.Workspace(dev)
    lab = torch.empty((n,), dtype=torch.int32, device=dev)
    steps_n = args.steps if headline else min(args.steps, 20)
    n_regions = 5 if headline else 3

    def sync_time(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        r = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, r

    fit = None
    if is_assign:
        y = w.y.to(dev)
        md = torch.empty((n,), dtype=torch.float32, device=dev)
        first_ms, _ = sync_time(lambda: _native.assign(x, y, lab, md, ws))

        def steps(count):
            for _ in range(count):
                _native.assign(x, y, lab, md, ws)

        def kernel_only():
            _native.assign(x, y, lab, md, ws)
    else:
        xd = ht.array(x, split=0)
        c0 = ht.array(w.init.to(dev))
        t_iter = w.max_iter

        def one_fit():
            return ht.cluster.KMeans(n_clusters=k, init=c0, max_iter=t_iter, tol=0.0).fit(xd)

        first_ms, km = sync_time(one_fit)
        del km
        # the loop of KMeans.fit in the long run: per iteration one hkm_lloyd_step_f32 and a 4-byte read of the
        # shift (tol = -1: the host looks at every shift, as with tol = 0, but never stops early)
        loop = LloydLoop(x, w.init.to(dev), ws)
        shift = torch.zeros((), dtype=torch.float32, device=dev)
        c_tmp = torch.empty_like(loop.centers)

        def steps(count):
            assert loop.run(count, -1.0) == count
            loop.labels  # what fit() returns: for narrow shapes this is the one pass that stores labels

        def kernel_only():
            if kernel.startswith("lloyd_"):
                # one-sweep shapes: the step IS the dominant kernel plus a few finishing launches of some 10 us
                # (without storing labels where the fit loop does not store them either)
                _native.lloyd_step(x, loop.centers, c_tmp, None if loop.lazy_labels else lab, shift, None, ws)
            else:
                _native.assign(x, loop.centers, lab, None, ws)

    # a device that has been idle runs its first ~25 ms of work up to 30 % slower: if fewer than 30
    # warm-up steps are asked for, the difference is run before them (untimed, reported as "prewarm")
    prewarm = max(0, 30 - args.warmup)
    if prewarm:
        steps(prewarm)
    steps(args.warmup)
    regions = []
    for _ in range(n_regions):
        t_ms, _ = sync_time(lambda: steps(steps_n))
        regions.append(t_ms * 1e-3)
    elapsed = sorted(regions)[len(regions) // 2]

    # the dominant kernel alone: one more pass of the same steps with the library recording an event pair
    # on the launch stream right around that kernel (and nothing else)
    benchhooks.profile_enable(True)
    if is_assign:
        steps(min(steps_n, 512))
    else:
        assert loop.run(min(steps_n, 512), -1.0) == min(steps_n, 512)
    torch.cuda.synchronize()
    kern = benchhooks.profile_collect()
    benchhooks.profile_enable(False)
    kern_ms = sum(kern) / len(kern)

    # the fits, warm: R of them one after the other, each between two synchronisations
    if not is_assign:
        n_fits = max(5, -(-args.steps // t_iter)) if headline else 5
        one_fit()
        times = []
        for _ in range(n_fits):
            t_ms, km = sync_time(one_fit)
            times.append(t_ms)
        fit_ms = sorted(times)[len(times) // 2]
        # the timed fit's own result: every row labelled, and the two-pass means of its labels are its centroids
        lab64 = km.labels_.larray.view(-1)
        counts = torch.bincount(lab64, minlength=k)
        c_chk = torch.empty((k, d), dtype=torch.float32, device=dev)
        _native.update(x, lab64.to(torch.int32), c_chk, None, ws)
        cen = km.cluster_centers_.larray
        err = float((c_chk - cen).abs().max() / cen.abs().max().clamp_min(1e-30))
        ok = int(counts.sum()) == n and int(lab64.min()) >= 0 and int(lab64.max()) < k and err <= 1e-6
        fit = {"fit_ms": round(fit_ms, 4), "fit_ms_min": round(min(times), 4), "fit_ms_max": round(max(times), 4),
               "fits_timed": n_fits, "first_fit_ms": round(first_ms, 3), "n_iter": int(km.n_iter_), "max_iter": t_iter,
               "tol": 0.0, "value_fit": round(n * km.n_iter_ / (fit_ms * 1e-3), 1),
               "checked": bool(ok), "check_centroid_rel_err": float(f"{err:.3g}"),
               "inertia": float(km.inertia_)}
        del km, lab64, c_chk
    else:
        # the assignment's own result on a sample of rows, against float64 distances
        idx = torch.arange(0, n, max(1, n // 512), device=dev)[:512]
        d2 = torch.cdist(x[idx].double(), y.double()) ** 2
        best = d2.min(dim=1).values
        mine = d2.gather(1, lab[idx].long().view(-1, 1)).view(-1)
        res = 4.0 * 1.1920929e-07 * ((x[idx].double() ** 2).sum(1) + (y.double() ** 2).sum(1).max())
        ok = bool(((mine - best) <= 1e-5 * best + res).all()) and bool(((md[idx].double() - mine).abs() <= 1e-4 * mine + res).all())
        fit = {"first_call_ms": round(first_ms, 3), "checked": ok}

    flops = 2.0 * n * k * d
    nbytes = float(n) * (4 * d + 4) if not is_assign else float(n) * (4 * d + 8) + 4.0 * k * d
    tf = flops / (kern_ms * 1e-3) / 1e12
    gbs = nbytes / (kern_ms * 1e-3) / 1e9
    # a free shape is priced against the matrix pipe where the matrix cores run it, against HBM otherwise
    mfma_bound = config in MFMA_BOUND or (config == "shape" and kernel.startswith(("lloyd_mfma", "mfma")))
    if mfma_bound:
        roof = {"bound": "mfma", "achieved": round(tf, 3), "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)}
    else:
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}
    roof["kernel"] = kernel
    roof["kernel_ms"] = round(kern_ms, 4)
    roof["kernel_launches_timed"] = len(kern)
    traffic, traffic_source = _traffic(config, w.name, args.scale, args.shape)
    roof["traffic"] = traffic
    # the counters' bytes over the same kernel time: what the memory system really moved, against its peak
    roof["traffic_frac"] = round(traffic / (kern_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4) if traffic else None
    if kernel in ("lloyd_mfma_resident", "mfma_resident"):
        # which of the two launch geometries of the resident kernels ran, and whether that is the verdict of the
        # library's trial on this device (taken on the steps above) or the default / HKM_POINT_BLOCKS
        pb, tuned = benchhooks.point_blocks(d)
        roof["point_blocks_per_wave"] = pb
        roof["point_blocks_measured_here"] = tuned
    value = (n * fit["n_iter"] / (fit["fit_ms"] * 1e-3)) if not is_assign else n * steps_n / elapsed
    res = {"w": w, "x": x, "roof": roof, "fit": fit, "value": value, "elapsed": elapsed, "regions": regions,
           "steps": steps_n, "prewarm": prewarm, "t_gen": t_gen, "kernel": kernel, "kernel_only": kernel_only,
           "steps_fn": steps, "mfma_bound": mfma_bound, "traffic_source": traffic_source, "tf": tf, "gbs": gbs,
           "n": n, "d": d, "k": k}
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--config", default="all", choices=["all", "c1", "c2", "c3", "c4", "c5"],
                    help="all (default): the headline workload c3 in full, then the other four workloads' figures "
                         "in the same line under `configs`; cN: that workload alone, in full")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink N (testing only; invalidates the figure)")
    ap.add_argument("--shape", type=int, nargs=3, metavar=("N", "D", "K"), default=None,
                    help="time the Lloyd step on K equal blobs of this shape instead of a named workload "
                         "(not a headline figure: no CPU baseline, no traffic)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--probe", action="store_true",
                    help="run the hardware microbenchmarks (matrix-pipe throughput alone and with interleaved "
                         "vector / scalar instructions; copy, read and fill bandwidth) instead of a workload")
    ap.add_argument("--estimator", default="kmeans", choices=["kmeans", "kmedians", "cdist", "init", "knn", "silhouette"],
                    help="kmedians: the Manhattan-metric sibling on the same data; cdist: the full-matrix "
                         "public cdist on rows of c2; init: the k-means|| initialiser; knn: k nearest rows + label vote on rows of c2; silhouette: silhouette_samples on 100 000 rows of c3 (none is the headline metric)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        return 2

    import torch

    from heat_amd import _native
    from heat_amd.utils import synthetic

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    _native.load()
    if args.probe:
        return run_probe()
    dev = torch.device("cuda:0")

    if args.estimator != "kmeans":
        cfg = "c3" if args.config == "all" else args.config
        t_gen = time.perf_counter()
        w = synthetic.CONFIGS[cfg](args.scale)
        t_gen = time.perf_counter() - t_gen
        x = w.x.to(dev)
        args.config = cfg
        fn = {"kmedians": bench_kmedians, "cdist": bench_cdist, "init": bench_init, "knn": bench_knn,
              "silhouette": bench_silhouette}[args.estimator]
        return fn(args, w, x, t_gen)

    all_configs = args.config == "all" and not args.shape
    head_cfg = "c3" if args.config == "all" else args.config
    if args.shape:
        args.no_cpu_baseline = True
    m = measure(args, head_cfg, headline=True)
    w, x, roof, n, d, k = m["w"], m["x"], m["roof"], m["n"], m["d"], m["k"]
    kernel_only = m["kernel_only"]
    is_assign = head_cfg == "c2" and not args.shape

    # the whole step (every launch of it, no host read) between two events on the same stream
    ev_ms = []
    for _ in range(m["steps"]):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        kernel_only()
        e1.record()
        torch.cuda.synchronize()
        ev_ms.append(e0.elapsed_time(e1))
    roof["step_ms_events"] = round(sum(ev_ms) / len(ev_ms), 4)
    roof["mfma_frac"] = round(m["tf"] / PEAK_FP32_MFMA_TFLOPS, 4)
    roof["hbm_frac"] = round(m["gbs"] / PEAK_HBM_GBS, 4)
    # The shader clock while the dominant kernel runs back to back (best effort: the driver's own
    # figure, read from sysfs between batches of launches; None where the file is not there).  `peak`
    # assumes 2400 MHz; some chips hold less under the matrix-core kernels, and then `frac` is lower
    # by that ratio although the kernel does the same work per clock.
    roof["sclk_mhz_under_load"] = sclk_under_load(lambda: [kernel_only() for _ in range(20)])
    if m["mfma_bound"]:
        roof["mfma_alone_tflops_this_chip"] = round(mfma_alone_tflops(), 1)
    roof["traffic_source"] = m["traffic_source"]

    # Not the headline: the same timed loop with the opt-in split-bf16 products (HKM_PRODUCTS=bf16x3;
    # every product still accurate to fp32, evaluated as six bf16 partial products on the bf16 matrix
    # cores), where that path exists.  `value` above is the all-fp32 default.
    alt = None
    if m["kernel"] == "lloyd_mfma_resident" and 16 < d <= 32 and not is_assign:
        os.environ["HKM_PRODUCTS"] = "bf16x3"
        try:
            m["steps_fn"](30)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            m["steps_fn"](m["steps"])
            torch.cuda.synchronize()
            t_alt = time.perf_counter() - t1
        finally:
            os.environ.pop("HKM_PRODUCTS", None)
        alt = {"env": "HKM_PRODUCTS=bf16x3", "ms_per_step": round(t_alt / m["steps"] * 1e3, 4),
               "value": round(n * m["steps"] / t_alt, 1), "unit": "points*iter/s",
               "products": "3-way split bf16 operands, 6 partial products, fp32 accumulate"}

    cpu = None
    if not args.no_cpu_baseline:
        from oracle import heat_oracle as orc

        div = CPU_SAMPLE_DIV[head_cfg]
        ns = max(n // div, min(n, 4 * k))
        xs = w.x[:ns].contiguous()
        torch.set_num_threads(os.cpu_count() or 1)
        t1 = time.perf_counter()
        if is_assign:
            its = 1
            orc.assign_to_cluster_literal(xs, w.y)
        else:
            its = w.max_iter if head_cfg == "c1" else 2  # c1 is small enough for its whole fit
            orc.kmeans_fit(xs, w.init, its, None, literal=True)
        t_cpu = time.perf_counter() - t1
        cpu = {"value": round(ns * its / t_cpu, 1), "unit": "points*iter/s", "cores": torch.get_num_threads(),
               "kind": "port",
               "sample": f"first {ns} rows of the same data, {its} iteration(s), op-for-op restatement of "
                         f"Heat's torch-CPU sequence, {t_cpu:.1f} s"}

    fit = m["fit"]
    steady = {"value": round(n * m["steps"] / m["elapsed"], 1), "ms_per_step": round(m["elapsed"] / m["steps"] * 1e3, 4),
              "ms_per_step_min": round(min(m["regions"]) / m["steps"] * 1e3, 4),
              "ms_per_step_max": round(max(m["regions"]) / m["steps"] * 1e3, 4),
              "timed_regions": len(m["regions"]), "steps_per_region": m["steps"]}
    out = {
        "metric": "KMeans Lloyd points*iter/s" if not is_assign else "cdist+argmin points/s",
        "value": round(m["value"], 1),
        "unit": "points*iter/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(fit["fit_ms"] / fit["n_iter"], 4) if not is_assign else steady["ms_per_step"],
        "value_is": ("N * n_iter_ / wall time of KMeans(n_clusters=K, init=C0, max_iter=T, tol=0).fit(x), median of the "
                     "timed fits (see fit); steady_state is the same step in a long loop") if not is_assign
                    else "N / wall time of one fused distance+argmin call in a loop",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {m['t_gen']:.1f} s, resident in HBM before timing)",
        "config": {"workload": w.name, "N": n, "D": d, "K": k, "scale": args.scale, "prewarm": m["prewarm"]},
        "fit": fit,
        "steady_state": steady,
        "roofline": roof,
        "cpu_baseline": cpu,
    }
    if alt:
        out["split_products"] = alt
    if all_configs:
        # the other four workloads, figures only (their full lines: bench.py --config cN)
        del m, x, w, kernel_only
        torch.cuda.empty_cache()
        others = {}
        for cfg in ("c1", "c2", "c4", "c5"):
            mm = measure(args, cfg, headline=False)
            f, r = mm["fit"], mm["roof"]
            e = {"workload": mm["w"].name, "value": round(mm["value"], 1),
                 "unit": "points/s" if cfg == "c2" else "points*iter/s",
                 "ms_per_step_steady": round(mm["elapsed"] / mm["steps"] * 1e3, 4),
                 "kernel": r["kernel"], "kernel_ms": r["kernel_ms"], "bound": r["bound"], "frac": r["frac"],
                 "traffic": r["traffic"], "traffic_frac": r["traffic_frac"], "checked": f["checked"]}
            for key in ("fit_ms", "first_fit_ms", "n_iter", "first_call_ms"):
                if key in f:
                    e[key] = f[key]
            others[cfg] = e
            del mm
            torch.cuda.empty_cache()
        out["configs"] = others
    print(json.dumps(out))
    return 0 if (fit["checked"] and all(e["checked"] for e in out.get("configs", {}).values())) else 1


if __name__ == "__main__":
    sys.exit(main())
