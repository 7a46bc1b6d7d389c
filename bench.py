#!/usr/bin/env python3
"""
Benchmark of the k-means Lloyd step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3] [--no-cpu-baseline]

A step is one Lloyd iteration (labels, per-cluster means, centroid shift) over the whole synthetic
data set, issued exactly as KMeans.fit issues it: one hkm_lloyd_step_f32 call, then the host reads
the 4-byte shift.  Inputs are resident in HBM before the timed region.  Prints ONE JSON line.

value      points*iterations / s over the timed region (wall clock, synchronised both sides)
roofline   the dominant kernel (fused distance+argmin) timed with events on the launch stream:
           algorithmic flops 2*N*K*D (MFMA-bound shapes) or bytes N*(4D+4) (HBM-bound shapes) per
           launch divided by its mean duration
cpu_baseline  the CPU restatement of the reference's op sequence (oracle/, torch CPU, all host
           threads) on a bounded row sample of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK_FP32_MFMA_TFLOPS = 157.3
# configs that are bound by the fp32 matrix pipe; the others stream X from HBM
MFMA_BOUND = {"c2", "c3", "c4"}
CPU_SAMPLE_DIV = {"c1": 1, "c2": 16, "c3": 32, "c4": 256, "c5": 128}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="c3", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--scale", type=float, default=1.0, help="shrink N (testing only; invalidates the figure)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: this build has no multi-GPU path (run with --gpus 1).", file=sys.stderr)
        return 2

    import torch

    import heat_amd as ht
    from heat_amd import _native
    from heat_amd.utils import synthetic

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    _native.load()
    dev = torch.device("cuda:0")

    t_gen = time.perf_counter()
    w = synthetic.CONFIGS[args.config](args.scale)
    t_gen = time.perf_counter() - t_gen
    n, d = w.x.shape
    k = w.k
    x = w.x.to(dev)
    kernel = _native.assign_kernel_name(n, d, k)
    ws = _native.Workspace(dev)
    lab = torch.empty((n,), dtype=torch.int32, device=dev)

    ev_ms = []
    if args.config == "c2":
        # assignment only: labels + min squared distance
        y = w.y.to(dev)
        md = torch.empty((n,), dtype=torch.float32, device=dev)

        def step():
            _native.assign(x, y, lab, md, ws)

        def kernel_only():
            _native.assign(x, y, lab, md, ws)
    else:
        c_cur = w.init.to(dev).clone()
        c_nxt = torch.empty_like(c_cur)
        shift = torch.zeros((), dtype=torch.float32, device=dev)
        state = {"cur": c_cur, "nxt": c_nxt}

        def step():
            _native.lloyd_step(x, state["cur"], state["nxt"], lab, shift, None, ws)
            state["cur"], state["nxt"] = state["nxt"], state["cur"]
            shift.item()  # the convergence test of KMeans.fit: a 4-byte read per iteration

        def kernel_only():
            _native.assign(x, state["cur"], lab, None, ws)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # dominant kernel alone, event-timed on the stream it is launched on (torch's current stream)
    fused_small_d = kernel == "valu_fused"
    for _ in range(args.steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step() if fused_small_d else kernel_only()
        e1.record()
        torch.cuda.synchronize()
        ev_ms.append(e0.elapsed_time(e1))
    kern_ms = sum(ev_ms) / len(ev_ms)

    if args.config in MFMA_BOUND:
        flops = 2.0 * n * k * d
        achieved = flops / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_FP32_MFMA_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4)}
    else:
        nbytes = float(n) * (4 * d + 4)
        achieved = nbytes / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4)}
    roof["kernel"] = kernel
    roof["kernel_ms"] = round(kern_ms, 4)
    roof["traffic"] = None
    tfile = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tfile):
        with open(tfile) as f:
            roof["traffic"] = json.load(f).get(w.name)

    cpu = None
    if not args.no_cpu_baseline:
        from oracle import heat_oracle as orc

        div = CPU_SAMPLE_DIV[args.config]
        ns = max(n // div, min(n, 4 * k))
        xs = w.x[:ns].contiguous()
        torch.set_num_threads(os.cpu_count() or 1)
        t1 = time.perf_counter()
        if args.config == "c2":
            its = 1
            orc.assign_to_cluster_literal(xs, w.y)
        else:
            its = 2
            orc.kmeans_fit(xs, w.init, its, None, literal=True)
        t_cpu = time.perf_counter() - t1
        cpu = {"value": round(ns * its / t_cpu, 1), "unit": "points*iter/s", "cores": torch.get_num_threads(),
               "kind": "port",
               "sample": f"first {ns} rows of the same data, {its} iteration(s), op-for-op restatement of "
                         f"Heat's torch-CPU sequence, {t_cpu:.1f} s"}

    out = {
        "metric": "KMeans Lloyd points*iter/s" if args.config != "c2" else "cdist+argmin points/s",
        "value": round(n * args.steps / elapsed, 1),
        "unit": "points*iter/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": f"synthetic (seed {w.seed}, generated on CPU in {t_gen:.1f} s, resident in HBM before timing)",
        "config": {"workload": w.name, "N": n, "D": d, "K": k, "scale": args.scale},
        "roofline": roof,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
