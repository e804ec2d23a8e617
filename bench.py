#!/usr/bin/env python3
"""Lloyd-iteration throughput of the gfx950 k-means engine on one MI355X.

A step is one Lloyd iteration (fused distance+argmin pass, then the centroid
update) over the whole resident data set. The default workload is the headline
shape: 10,000,000 x 32 float32 Gaussian blobs, k = 256, seeded-random row
initialisation. Prints one JSON line.

    python bench.py [--gpus 1] [--steps 30] [--warmup 3] [--workload C3] [--no-traffic]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from h2o4gpu_amd import datasets  # noqa: E402
from h2o4gpu_amd.libs import kmeans_hip  # noqa: E402

PEAK_HBM_GBPS = 8000.0
PEAK_MFMA_TFLOPS = {"f32": 157.3, "f64": 78.6}
PEAK_BF16_TFLOPS = 2500.0  # dense bfloat16 matrix peak (option fp32_split)

WORKLOAD_TEXT = {
    "C1": "Gaussian blobs, seeded-random row start",
    "C2": "Gaussian blobs (Dirichlet sizes), seeded-random row start",
    "C3": "Gaussian blobs (equal sizes), seeded-random row start",
    "C4": "Gaussian blobs + 10% uniform outliers, k-means++ start from a fixed seed",
    "C5": "image-like rows (70% zeros, integers 1..255), seeded-random row start",
}


def measure_traffic(argv_tail, timeout_s=240):
    """HBM bytes per launch of the Lloyd-step kernel of this very workload, measured now:
    two child runs of this script under `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE, KiB
    per dispatch), each scaled by what the same counter reads for the library's plain copy
    kernel of 1 GiB in the same run. Must be called before this process touches the GPU.
    Returns (bytes or None, details)."""
    import csv
    import glob
    import shutil
    import subprocess
    import tempfile
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(rocprof):
        return None, {"skipped": "rocprofv3 not found"}
    if any(key.startswith(("ROCPROF", "ROCP_")) for key in os.environ):
        return None, {"skipped": "this run is itself being profiled"}
    details = {}
    total = 0.0
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        tmp = tempfile.mkdtemp(prefix="km_traffic_", dir="/tmp")
        cmd = [rocprof, "--pmc", counter, "--output-format", "csv", "-d", tmp, "-o", "x", "--",
               sys.executable, os.path.abspath(__file__), "--traffic-child"] + argv_tail
        env = dict(os.environ, TMPDIR="/tmp")
        try:
            proc = subprocess.run(cmd, cwd="/tmp", env=env, stdout=subprocess.PIPE,
                                  stderr=subprocess.STDOUT, timeout=timeout_s)
            files = glob.glob(os.path.join(tmp, "**", "*counter_collection.csv"), recursive=True)
            if proc.returncode != 0 or not files:
                return None, {"skipped": "%s pass failed (rc %d)" % (counter, proc.returncode)}
            per_kernel = {}
            for row in csv.DictReader(open(files[0])):
                if row["Counter_Name"] != counter:
                    continue
                per_kernel.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
        except Exception as exc:  # pylint: disable=broad-except
            return None, {"skipped": "%s pass: %r" % (counter, exc)}
        finally:
            shutil.rmtree(tmp, ignore_errors=True)
        copy = [v for name, v in per_kernel.items() if "copy_probe_kernel" in name]
        step = [(len(v), name, v) for name, v in per_kernel.items()
                if ("assign_" in name or "lloyd_valu" in name or "lloyd_longrow" in name)]
        if not copy or not step:
            return None, {"skipped": "%s pass: kernels not found" % counter}
        # the Lloyd-step kernel is the assign/step kernel with the most dispatches
        _, name, vals = max(step)
        copy_kib = sum(copy[0]) / len(copy[0])
        factor = (1 << 20) / copy_kib            # the copy kernel reads and writes 1 GiB = 2^20 KiB
        kib = sum(vals) / len(vals)
        details[counter] = {"kernel": name.split("(")[0][-90:], "raw_kib_per_dispatch": kib,
                            "copy_kernel_raw_kib": copy_kib, "scale": factor, "dispatches": len(vals)}
        total += kib * factor * 1024.0
    return total, details


def load_workload(args, dtype):
    """Rows, k, seed and the benchmark's iteration count of the workload the arguments name: one of
    the five configurations, or (--shape) unit-variance noise of any shape, drawn once as a block of
    16M values and repeated (a sweep over shapes should not wait for a generator)."""
    if args.shape:
        n, d, k = (int(v) for v in args.shape.lower().split("x"))
        base = np.random.default_rng(1).standard_normal(1 << 24).astype(np.float32)
        reps = -(-(n * d) // base.size)
        X = np.ascontiguousarray(np.tile(base, reps)[:n * d].reshape(n, d).astype(dtype))
        return X, k, 1, 5
    X, k, _ = datasets.make(args.workload, args.scale, dtype)
    return X, k, datasets.SHAPES[args.workload][3], datasets.SHAPES[args.workload][4]


def traffic_child(args):
    """The run the counters are read from: a few Lloyd steps of the workload plus the copy
    kernel that calibrates the counter."""
    dtype = np.float32 if args.dtype == "f32" else np.float64
    X, k, seed, _ = load_workload(args, dtype)
    n, d = X.shape
    h = kmeans_hip.Handle(n, d, k, dtype)
    h.set_data(X)
    h.set_centroids(datasets.seeded_row_init(X, k, seed))
    h.set_option("assign", args.assign)
    if args.no_fuse:
        h.set_option("fuse", 0)
    if args.exact_argmin:
        h.set_option("exact_argmin", 1)
    if args.fp32_split is not None:
        h.set_option("fp32_split", args.fp32_split)
    h.iterate(4)
    h.assign()
    h.close()
    kmeans_hip.copy_probe(1 << 30, 2)
    return 0


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def cpu_baseline(X, C0, iters, budget_s=12.0):
    """The CPU restatement (oracle port) timed on this host's cores: full Lloyd
    iterations (assign + update) over all rows, all hardware threads. With iters == 0
    it runs whole iterations until `budget_s` seconds have passed (at least 3)."""
    from oracle import load_oracle
    orc = load_oracle()
    threads = min(os.cpu_count() or 1, orc.max_threads)
    C = C0.copy()
    done = 0
    t0 = time.perf_counter()
    while True:
        labels = orc.assign(X, C, threads=threads)
        C, _ = orc.update(X, labels, C, threads=threads)
        done += 1
        dt = time.perf_counter() - t0
        if iters > 0 and done >= iters:
            break
        if iters <= 0 and done >= 3 and (dt >= budget_s or done >= 200):
            break
    return {"value": done / dt, "unit": "iter/s", "cores": threads, "kind": "port",
            "sample": "%d full Lloyd iterations (assign+update) over all %d rows, "
                      "C++/OpenMP restatement of the reference semantics" % (done, X.shape[0]),
            "seconds": dt}


def sklearn_baseline(X, C0, sample_rows, iters=5):
    """The reference's CPU fallback (kmeans.py:713-750 hands the fit to scikit-learn's
    KMeans): Lloyd from the same initial centroids on the first `sample_rows` rows, timed
    around fit(); per-iteration time = wall / n_iter_ (validation, centring and the final
    relabel included), scaled to the full row count."""
    try:
        import sklearn
        from sklearn.cluster import KMeans as SkKMeans
    except Exception as exc:  # not installed on this box
        return {"available": False, "reason": repr(exc)}
    import warnings
    n = X.shape[0]
    m = min(n, sample_rows)

    def timed(rows, max_iter):
        est = SkKMeans(n_clusters=C0.shape[0], init=C0.copy(), n_init=1, max_iter=max_iter, tol=0.0,
                       algorithm="lloyd")
        t0 = time.perf_counter()
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            est.fit(X[:rows])
        return time.perf_counter() - t0, int(est.n_iter_)

    timed(min(m, 50_000), 1)  # thread-pool start-up and lazy imports
    dt, n_iter = timed(m, iters)
    per_iter = dt / max(n_iter, 1) * (float(n) / m)
    return {"available": True, "version": sklearn.__version__, "value": 1.0 / per_iter,
            "unit": "iter/s", "cores": os.cpu_count() or 1,
            "kind": "reference CPU fallback (scikit-learn)",
            "sample": "KMeans(init=<same centroids>, n_init=1, max_iter=%d, tol=0, algorithm='lloyd')"
                      ".fit on the first %d rows: wall / n_iter_ (%d), scaled by %d/%d rows"
                      % (iters, m, n_iter, n, m),
            "seconds": dt}


def c_abi_fit(X, C0, iters):
    """One whole fit through the reference's C entry point (host pointers in, host
    results out): upload, row norms, `iters` Lloyd iterations, final relabel, download."""
    from h2o4gpu_amd.libs import ch2o4gpu_gpu as shim
    n, d = X.shape
    k = C0.shape[0]
    fn = shim.make_ptr_float_kmeans if X.dtype == np.float32 else shim.make_ptr_double_kmeans
    cent = np.empty(k * d, X.dtype)
    lab = np.empty(n, np.int32)
    t0 = time.perf_counter()
    rc = fn(0, 0, 0, 0, 1, n, d, k, iters, 2, 0.0, X.reshape(-1), C0.reshape(-1), cent, lab)
    dt = time.perf_counter() - t0
    return {"status": int(rc), "iterations": iters, "seconds": dt,
            "note": "make_ptr_*_kmeans with init_from_data=2: pageable host memory in, "
                    "malloc'ed results out"}


def seeding_seconds(X, k, seed=7):
    """The reference's default start (k-means||, then its host k-means++ over the candidates)
    on rows already resident: not part of a step, reported beside it."""
    from h2o4gpu_amd.libs import kmeans_hip
    n, d = X.shape
    with kmeans_hip.Handle(n, d, k, X.dtype) as h:
        h.set_data(X)
        h.init_parallel(seed)  # (first call: lazy set-up)
        t0 = time.perf_counter()
        h.init_parallel(seed + 1)
        dt = time.perf_counter() - t0
        info = h.parallel_seed_info()
    return {"seconds": dt, "candidates": int(len(info["cand_rows"])),
            "note": "init_from_data=1 on resident rows: rounds of k-means||, weights, k picks"}


def hbm_probes(nbytes=1 << 30, reps=10):
    """What this device's memory system delivers for plain streaming kernels over 1 GiB: the
    measured roof beside the 8 TB/s datasheet figure."""
    out = {"bytes": nbytes}
    for kind, moved in (("read", 1.0), ("write", 1.0), ("copy", 2.0), ("memcpy", 2.0)):
        ms = kmeans_hip.bandwidth_probe(kind, nbytes, reps)
        out[kind + "_gbps"] = moved * nbytes / (ms * 1e-3) / 1e9
    return out


def extra_step(workload, scale, steps, warmup=2):
    """One more shape timed in this process after the headline one, the same way: `steps`
    Lloyd steps (assign + update) on resident rows between stream events, then again with an
    event pair round every launch for the dominant kernel's average. float32."""
    t0 = time.perf_counter()
    X, k, _ = datasets.make(workload, scale, np.float32)
    n, d = X.shape
    gen_s = time.perf_counter() - t0
    seed = datasets.SHAPES[workload][3]
    with kmeans_hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        if workload == "C4":
            h.init_plusplus(seed)   # the benchmark's start for this shape: k-means++, fixed seed
        else:
            h.set_centroids(datasets.seeded_row_init(X, k, seed))
        variant = h.assign_variant()
        h.iterate(warmup)
        h.timer_start()
        h.iterate(steps)
        ms_step = h.timer_stop() / steps
        h.profile(True)
        h.iterate(steps)
        kern = {}
        for name in ("assign", "accumulate", "assign_accumulate", "finalize"):
            cnt, ms = h.kernel_time(name)
            if cnt:
                kern[name] = ms / cnt
        h.profile(False)
    dom = "assign_accumulate" if "assign_accumulate" in kern else "assign"
    out = {"workload": "%s generator: %d x %d f32, k=%d" % (workload, n, d, k), "assign_variant": variant,
           "steps": steps, "ms_per_step": ms_step, "kernel": "%s (%s)" % (dom, variant),
           "kernel_avg_ms": kern[dom], "kernels_avg_ms": {a: round(b, 5) for a, b in kern.items()},
           "generation_seconds": gen_s}
    if variant == "valu":
        # the iteration's algorithmic bytes: rows read once, labels written once, centroids in and out
        nbytes = float(n) * d * 4 + 4.0 * n + 2.0 * k * d * 4
        gbps = nbytes / (kern[dom] * 1e-3) / 1e9
        out.update({"bound": "hbm", "algorithmic_bytes": nbytes, "achieved": gbps, "peak": PEAK_HBM_GBPS,
                    "unit": "GB/s", "frac": gbps / PEAK_HBM_GBPS})
    else:
        tf = 2.0 * n * k * d / (kern[dom] * 1e-3) / 1e12
        out.update({"bound": "mfma", "algorithmic_flops": 2.0 * n * k * d, "achieved": tf,
                    "peak": PEAK_MFMA_TFLOPS["f32"], "unit": "TFLOP/s", "frac": tf / PEAK_MFMA_TFLOPS["f32"]})
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C3", choices=sorted(datasets.SHAPES))
    ap.add_argument("--scale", type=float, default=1.0, help="row-count scale (1.0 = full shape)")
    ap.add_argument("--shape", default=None, metavar="ROWSxCOLSxK",
                    help="instead of a configuration: unit-variance noise of this shape, seeded-random row start "
                         "(for sweeps over shapes; the bench line then names the shape as its workload)")
    ap.add_argument("--dtype", default="f32", choices=["f32", "f64"])
    ap.add_argument("--assign", default="auto", choices=sorted(kmeans_hip.ASSIGN_VARIANTS))
    ap.add_argument("--exact-argmin", action="store_true",
                    help="float32 matrix-core kernels: compare float distances instead of 16-ulp keys")
    ap.add_argument("--fp32-split", type=int, default=None, choices=[0, 6, 9],
                    help="float32 matrix-core kernels: dot products as this many bfloat16 products per "
                         "feature pair on the bfloat16 matrix pipe (9: every product exact)")
    ap.add_argument("--no-fuse", action="store_true",
                    help="keep assignment and accumulation as separate kernels")
    ap.add_argument("--transform-rows", type=int, default=0,
                    help="also time transform (full distance matrix) on this many held-out rows (C5)")
    ap.add_argument("--operands", default="generator", choices=["generator", "zeros", "ones", "normal"],
                    help="replace the values of the workload's rows (same shape, same kernels, same "
                         "instruction stream) by zeros, ones or unit-variance noise: shows how far the "
                         "chip's clock, and with it the kernel's time, follows the bit patterns it works on")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-iters", type=int, default=0, help="CPU baseline iterations (0 = about 12 s worth)")
    ap.add_argument("--sklearn-rows", type=int, default=10_000_000,
                    help="rows of the workload the scikit-learn leg runs on")
    ap.add_argument("--no-traffic", action="store_true",
                    help="skip the two rocprofv3 counter passes behind roofline.traffic")
    ap.add_argument("--traffic-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--no-end-to-end", dest="end_to_end", action="store_false",
                    help="skip the whole fit through make_ptr_*_kmeans (upload included, field c_abi_fit)")
    ap.add_argument("--end-to-end", dest="end_to_end", action="store_true", help=argparse.SUPPRESS)
    ap.set_defaults(end_to_end=True)
    ap.add_argument("--no-extras", dest="extras", action="store_false",
                    help="skip the two extra shapes timed after the headline one (the compute-bound "
                         "distance step at 2M x 256, k = 1024 and the bandwidth-bound step at 10M x 16, k = 8)")
    ap.set_defaults(extras=True)
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported "
              "(collectives and sharding are not part of this build)" % args.gpus, file=sys.stderr)
        return 2
    if args.traffic_child:
        return traffic_child(args)
    # the counter passes run in child processes, before this process initialises the GPU
    traffic, traffic_details = None, {"skipped": "--no-traffic"}
    if not args.no_traffic:
        tail = ["--workload", args.workload, "--scale", str(args.scale), "--dtype", args.dtype,
                "--assign", args.assign] + (["--shape", args.shape] if args.shape else []) + \
               (["--no-fuse"] if args.no_fuse else []) + \
               (["--exact-argmin"] if args.exact_argmin else []) + \
               (["--fp32-split", str(args.fp32_split)] if args.fp32_split is not None else [])
        t0 = time.perf_counter()
        traffic, traffic_details = measure_traffic(tail)
        log("traffic passes: %s in %.1f s" % ("%.4g bytes per launch" % traffic if traffic else
                                              traffic_details.get("skipped"), time.perf_counter() - t0))
    if kmeans_hip.device_count() < 1:
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 3

    dtype = np.float32 if args.dtype == "f32" else np.float64
    t0 = time.perf_counter()
    X, k, seed, fit_iters = load_workload(args, dtype)
    n, d = X.shape
    if args.operands != "generator":
        if args.operands == "normal":
            X = np.random.default_rng(seed).standard_normal(X.shape, dtype=dtype)
        else:
            X = np.full(X.shape, 0.0 if args.operands == "zeros" else 1.0, dtype)
    C0 = datasets.seeded_row_init(X, k, seed)
    wname = "noise %s" % args.shape if args.shape else args.workload
    log("generated %s: %d x %d %s, k=%d in %.1f s" % (wname, n, d, X.dtype, k, time.perf_counter() - t0))
    s = X.dtype.itemsize
    flops_per_iter = 2.0 * n * k * d
    bytes_per_iter = float(n) * d * s + 4.0 * n + 2.0 * k * d * s

    h = kmeans_hip.Handle(n, d, k, dtype)
    t0 = time.perf_counter()
    h.set_data(X)
    h2d_first_s = time.perf_counter() - t0  # includes the one-off pinned buffers and copy threads
    t0 = time.perf_counter()
    h.set_data(X)
    h2d_s = time.perf_counter() - t0
    if args.workload == "C4" and args.operands == "generator" and not args.shape:  # the benchmark text starts this shape from k-means++
        h.init_plusplus(seed)
        C0 = h.centroids()
    h.set_centroids(C0)
    h.set_option("assign", args.assign)
    if args.no_fuse:
        h.set_option("fuse", 0)
    if args.exact_argmin:
        h.set_option("exact_argmin", 1)
    if args.fp32_split is not None:
        h.set_option("fp32_split", args.fp32_split)
    variant = h.assign_variant()
    log("upload %.3f s (%.1f GB/s incl. pageable staging; first call of the process %.3f s); "
        "assign variant %s" % (h2d_s, n * d * s / h2d_s / 1e9, h2d_first_s, variant))

    # warm-up, then exactly K timed steps between stream events
    h.iterate(args.warmup)
    h.timer_start()
    h.timer_stop()
    h.timer_start()
    h.iterate(args.steps)
    ms_total = h.timer_stop()
    ms_step = ms_total / args.steps

    # per-kernel durations: same K steps again with an event pair round every launch
    h.profile(True)
    h.iterate(args.steps)
    kern = {}
    for name in ("assign", "accumulate", "assign_accumulate", "finalize", "post_update"):
        cnt, ms = h.kernel_time(name)
        if cnt:
            kern[name] = {"launches": cnt, "avg_ms": ms / cnt}
    h.profile(False)

    fused = "assign_accumulate" in kern
    dom = "assign_accumulate" if fused else "assign"
    assign_ms = kern[dom]["avg_ms"]
    tflops = flops_per_iter / (assign_ms * 1e-3) / 1e12
    peak = PEAK_MFMA_TFLOPS[args.dtype]
    mfma_bound = variant not in ("valu", "wave_row")   # (the kernels without matrix instructions stream X)
    if mfma_bound and "_bf16x" in variant:
        # the option that forms each float32 product from bfloat16 parts: the kernel executes
        # 6 or 9 times the algorithmic flop, on the bfloat16 matrix pipe, and is priced there
        products = int(variant[-1])
        roofline = {"bound": "mfma", "kernel": "%s (%s)" % (dom, variant), "achieved": products * tflops,
                    "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": products * tflops / PEAK_BF16_TFLOPS,
                    "traffic": traffic, "algorithmic_tflops": tflops,
                    "note": "%d bfloat16 products per float32 product, bfloat16 matrix peak" % products}
    elif mfma_bound:
        roofline = {"bound": "mfma", "kernel": "%s (%s)" % (dom, variant), "achieved": tflops,
                    "peak": peak, "unit": "TFLOP/s", "frac": tflops / peak, "traffic": traffic}
    else:
        # per row: the row read, the label written (inside a fit loop the fused step neither reads
        # the stored row norms nor writes the minimum distances)
        gbps = float(n) * (d * s + 4) / (assign_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": "%s (%s)" % (dom, variant), "achieved": gbps,
                    "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": gbps / PEAK_HBM_GBPS,
                    "traffic": traffic}
    iter_gbps = bytes_per_iter / (ms_step * 1e-3) / 1e9
    copy_bytes = 1 << 30
    copy_ms = kmeans_hip.copy_probe(copy_bytes, 10)
    try:
        probes = hbm_probes()
    except Exception as e:  # an extra: never the reason a bench line is missing
        probes = {"error": repr(e)}

    inertia = None
    h.assign()
    inertia = h.inertia()
    transform = None
    if args.transform_rows > 0:
        H = datasets.make_holdout(args.workload, args.transform_rows, dtype)
        h.transform(H[:1024])  # warm-up
        h.profile(True)
        t0 = time.perf_counter()
        h.transform(H)
        wall = time.perf_counter() - t0
        cnt, ms = h.kernel_time("transform")
        h.profile(False)
        tf = 2.0 * H.shape[0] * k * d / (ms * 1e-3) / 1e12
        transform = {"rows": int(H.shape[0]), "kernel_ms": ms, "launches": cnt, "tflops": tf,
                     "mfma_frac": tf / peak, "end_to_end_seconds": wall,
                     "output_bytes": float(H.shape[0]) * k * s}
    # the same steps with the float32 dot products on the bfloat16 matrix pipe (an option of
    # the matrix-core kernels, off by default; never part of `value`)
    split_leg = None
    if args.dtype == "f32" and variant in ("mfma_rowstat", "mfma_tiled"):  # (i.e. the main run was without it)
        h.set_option("fp32_split", 6)
        if h.assign_variant() == variant + "_bf16x6":
            h.set_centroids(C0)
            h.iterate(args.warmup)
            h.timer_start()
            h.iterate(args.steps)
            ms6 = h.timer_stop() / args.steps
            h.profile(True)
            h.iterate(args.steps)
            cnt6, kms6 = h.kernel_time(dom)
            h.profile(False)
            h.assign()
            split_leg = {"option": "fp32_split=6", "assign_variant": variant + "_bf16x6",
                         "ms_per_step": ms6, "iterations_per_s": 1000.0 / ms6,
                         "kernel_avg_ms": kms6 / max(cnt6, 1), "inertia": h.inertia(),
                         "note": "products of bfloat16 parts, float32 accumulation; same parity bars"}
        h.set_option("fp32_split", 0)
    h.close()

    out = {
        "metric": "lloyd_iterations_per_second", "value": 1000.0 / ms_step, "unit": "iter/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "%s: %d x %d %s, k=%d, %s; one step = assign + centroid update"
                               % (wname, n, d, args.dtype, k,
                                  "unit-variance noise, seeded-random row start" if args.shape
                                  else WORKLOAD_TEXT[args.workload]),
                   "rows": n, "cols": d, "k": k, "assign_variant": variant,
                   "operands": args.operands},
        "roofline": roofline,
        "traffic_measurement": traffic_details,
        "iteration": {"algorithmic_bytes": bytes_per_iter, "algorithmic_flops": flops_per_iter,
                      "gbps": iter_gbps, "hbm_frac": iter_gbps / PEAK_HBM_GBPS,
                      "tflops": flops_per_iter / (ms_step * 1e-3) / 1e12,
                      "mfma_frac": flops_per_iter / (ms_step * 1e-3) / 1e12 / peak},
        "kernels_avg_ms": {kname: round(v["avg_ms"], 5) for kname, v in kern.items()},
        "copy_probe_gbps": 2.0 * copy_bytes / (copy_ms * 1e-3) / 1e9,
        "hbm_probes": probes,
        "h2d_seconds": h2d_s,
        "h2d_seconds_first_call": h2d_first_s,
        "inertia": inertia,
    }
    if transform:
        out["transform"] = transform
    if split_leg:
        out["fp32_split"] = split_leg
    if args.extras and args.workload == "C3" and args.scale == 1.0 and args.dtype == "f32" and not args.shape:
        # the north star's two regimes under the same clock as the headline shape; extras, never
        # the reason a bench line is missing
        for key, wl, scale in (("c4_distance_step", "C4", 1.0), ("hbm_bound_step", "C1", 100.0)):
            try:
                t0 = time.perf_counter()
                # (the bandwidth-bound step is 0.15 ms: more steps and a longer warm-up, so that the
                # clock ramp after the idle time of the data generation is not what gets timed)
                out[key] = extra_step(wl, scale, 5 if wl == "C4" else 100, 2 if wl == "C4" else 20)
                if key == "hbm_bound_step" and "read_gbps" in probes:
                    out[key]["frac_of_read_probe"] = out[key]["achieved"] / probes["read_gbps"]
                    out[key]["frac_of_copy_probe"] = out[key]["achieved"] / probes["copy_gbps"]
                log("%s: %.4f ms per launch, %.3f of peak (%.1f s)" % (key, out[key]["kernel_avg_ms"],
                                                                         out[key]["frac"], time.perf_counter() - t0))
            except Exception as e:
                out[key] = {"error": repr(e)}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(X, C0, args.cpu_iters)
        out["cpu_reference_path"] = sklearn_baseline(X, C0, args.sklearn_rows)
    if args.end_to_end:
        out["c_abi_fit"] = c_abi_fit(X, C0, fit_iters)
        try:
            out["kmeans_parallel_seeding"] = seeding_seconds(X, k)
        except Exception as e:  # an extra: never the reason a bench line is missing
            out["kmeans_parallel_seeding"] = {"error": repr(e)}
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
