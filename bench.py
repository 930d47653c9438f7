#!/usr/bin/env python3
"""Benchmark of the BCPNN layer training step on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-other-configs]
  python bench.py --workload dense|mnist15x200|wide64|stl10|largest    one of the other configurations alone
  python bench.py --achievable-peaks                                   device-copy and matrix-core probes
  python bench.py --copy-calibration                                   known-size copies for counter scaling
  python bench.py --entry-point-rates                                  the per-function C entry points on their own
  python bench.py --passes                                             trace, weight and forward passes one by one
  python bench.py --pmc-summary DIR                                    text summary of rocprofv3 --pmc runs
  python bench.py --trace-summary DIR                                  per-kernel table of a rocprofv3 kernel trace

Headline workload: the MNIST-shaped 2-layer network, float32, batch 128, 60000 seeded
synthetic samples; input 784 pixels complementary-coded to 1568 units (~19% nonzero pixels, uniform
in (0,1]); hidden layer 30 hypercolumns x 100 minicolumns with a receptive-field mask of density 0.1;
10-class dense output layer.  A "step" is one structural-plasticity-layer training step on one
resident batch: forward x.W+b with per-hypercolumn softmax, Ci/Cj/Cij trace update, weight and bias
recompute, mask apply, and the mask rewiring at the reference's cadence (every 15th step of an epoch
after the first).  The timed region starts with the training set already in HBM.  The window of K steps
is timed several times; `value` and `ms_per_step` are the median window, `windows` holds the spread.

Prints one JSON line.  `value` is training samples/s; `roofline` describes the dominant kernel (the
fused trace+weight pass); `cpu_baseline` is the CPU restatement of the reference's cpu backend (its
OpenMP loop structure built with its flag set, the forward product through numpy's BLAS, numpy softmax)
timed on this host on a bounded number of the same steps, with a per-function split; `other_configs`
holds short runs of the other four configurations, each with its own roofline and CPU baseline.
"""
import argparse
import ctypes
import hashlib
import json
import os
import sys
import tempfile
import time

# thread placement of the CPU baseline's OpenMP loops (read when the OpenMP runtime first starts)
os.environ.setdefault("OMP_PROC_BIND", "close")
os.environ.setdefault("OMP_PLACES", "cores")

import numpy as np  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N_PIXELS, H, MC, N_OUT, BATCH, N_SAMPLES = 784, 30, 100, 10, 128, 60000
HP = dict(l1_taupdt=0.006908854922437549, l1_pmin=0.06195283356566607, l1_khalf=-139.02586632856327,
          l1_taubdt=0.02218100432360414, l1_density=0.1, l2_taupdt=0.0007449780036161324)
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f32": 157.3, "f64": 78.6}
PMC_PROFILE = os.path.join(ROOT, "profiles", "k_train_fused_mnist_f32_b128_pmc.txt")
KERNEL_SOURCES = ("sb_k_train.hpp", "sb_common.hpp")


def synthetic_dataset(n, seed=1001):
    rng = np.random.default_rng(seed)
    px = (1.0 - rng.random((n, N_PIXELS), dtype=np.float32)) * (rng.random((n, N_PIXELS), dtype=np.float32) < 0.19)
    x = np.concatenate([px, 1.0 - px], axis=1).astype(np.float32)
    y = np.zeros((n, N_OUT), dtype=np.float32)
    y[np.arange(n), rng.integers(0, N_OUT, n)] = 1.0
    return x, y


def initial_state(seed=0):
    """Layer state drawn in the reference's order from numpy's legacy global stream."""
    n, m = 2 * N_PIXELS, H * MC
    np.random.seed(seed)
    st = {
        "weights": (0.1 * np.random.randn(n, m)).astype(np.float32),
        "bias": (0.1 * np.random.rand(m)).astype(np.float32),
        "Ci": np.ones(n, dtype=np.float32),
        "Cj": np.full(m, 1.0 / MC, dtype=np.float32),
        "Cij": np.full((n, m), 1.0 / MC, dtype=np.float32),
        "kbi": np.ones(m, dtype=np.float32),
    }
    st["wmask"] = (np.random.rand(n, H) < HP["l1_density"]).astype(np.uint8)
    return st


def batch_plan(first_step, n_steps, nb):
    """Splits a run of consecutive steps into per-epoch ranges (epoch, first_batch, n_batches);
    epoch numbering starts at 1 so that the rewiring cadence is part of the measurement."""
    out = []
    step = first_step
    left = n_steps
    while left > 0:
        epoch, fb = 1 + step // nb, step % nb
        take = min(left, nb - fb)
        out.append((epoch, fb, take))
        step += take
        left -= take
    return out


def window_stats(times_s, samples, steps):
    """Median window (the reported one) and the spread over the timed windows of `steps` steps each."""
    order = np.argsort(times_s)
    mid = int(order[len(order) // 2])
    per_step = [1e3 * t / steps for t in times_s]
    return mid, {"count": len(times_s), "steps_each": steps, "ms_per_step_median": per_step[mid],
                 "ms_per_step_min": min(per_step), "ms_per_step_max": max(per_step)}


def n_windows(steps):
    """How often the window of `steps` steps is timed: about 3000 steps in all, 3 to 50 windows."""
    return int(min(50, max(3, -(-3000 // max(steps, 1)))))


def host_info():
    """CPU model, physical cores of the host and the threads the CPU baseline uses."""
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name") and model == "unknown":
                model = line.split(":", 1)[1].strip()
            elif line.startswith("physical id"):
                phys = line.split(":", 1)[1].strip()
            elif line.startswith("core id"):
                core = line.split(":", 1)[1].strip()
            elif not line.strip():
                if phys is not None and core is not None:
                    cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    blas = "unknown"
    try:
        cfg = np.show_config(mode="dicts")
        b = cfg.get("Build Dependencies", {}).get("blas", {})
        blas = f"{b.get('name', 'unknown')} {b.get('version', '')}".strip()
    except Exception:
        pass
    return {"cpu_model": model, "physical_cores_of_host": len(cores) or None, "logical_cpus_of_host": os.cpu_count(),
            "threads_used": threads, "numpy_blas": blas}


# ---------------------------------------------------------------------------------------- CPU baseline
def numpy_softmax(a, h, mc):
    """kernels_numpy.py:13-25 of the reference (what its cpu backend binds for the softmax)."""
    t = a.reshape(-1, h, mc)
    t = np.exp(t - t.max(axis=2, keepdims=True))
    return (t / t.sum(axis=2, keepdims=True)).reshape(a.shape)


def cpu_baseline(x, st, h, mc, batch, tau, dtype, budget_s, min_steps=1, rewire_period=15, warm=True):
    """The cpu backend's training step of one structural-plasticity layer on this host: forward product
    through numpy's BLAS (the reference calls cblas), numpy softmax (the reference's own), and the C
    restatement of its OpenMP kernels built with its flag set for the fused trace + weight pass, the
    regularised bias, the rewiring and the mask apply.  Batches in storage order, a rewiring every
    `rewire_period`-th step; at least min_steps timed steps, then until budget_s is used up."""
    from concurrent.futures import ThreadPoolExecutor
    from threadpoolctl import threadpool_limits
    from oracle import build as oracle_build
    from oracle.oracle import Oracle
    # the reference builds with -march=native: so does the baseline where this host has a compiler
    native = oracle_build.build_native(tempfile.mkdtemp(prefix="sb_cpu_baseline_"))
    o = Oracle(path=native) if native else Oracle(fast=True)
    march = "-march=native (built on this host)" if native else "-march=x86-64-v3 (no compiler on this host)"
    cthr = tau / 2
    info = host_info()
    full_batches = max(1, x.shape[0] // batch)
    split = {"forward_blas": 0.0, "softmax_numpy": 0.0, "traces_and_weights": 0.0, "bias": 0.0, "mask": 0.0}
    # The forward product runs numpy's BLAS kernel on every core, one column slice of W per thread with the
    # library's own threading off: its worker threads would otherwise keep spinning after each product
    # and take the cores from the OpenMP loops that follow (measured: those loops ran 2.4 times slower).
    threads = info["threads_used"]
    m = st["weights"].shape[1]
    cuts = [m * k // threads for k in range(threads + 1)]
    pool = ThreadPoolExecutor(threads)
    limit = threadpool_limits(limits=1, user_api="blas")

    def forward(xb):
        act = np.empty((xb.shape[0], m), dtype=dtype)

        def part(k):
            np.matmul(xb, st["weights"][:, cuts[k]:cuts[k + 1]], out=act[:, cuts[k]:cuts[k + 1]])
        list(pool.map(part, range(threads)))
        act += st["bias"]
        return act

    def step(i, timed):
        i = i % full_batches
        xb = x[i * batch:(i + 1) * batch]
        t = [time.perf_counter()]
        act = forward(xb)
        t.append(time.perf_counter())
        act = np.ascontiguousarray(numpy_softmax(act, h, mc), dtype=dtype)
        t.append(time.perf_counter())
        o.update_weights(st["Ci"], st["Cj"], st["Cij"], xb, act, tau, st["weights"], cthr)
        t.append(time.perf_counter())
        o.update_bias_regularized(st["bias"], st["kbi"], st["Cj"], cthr, HP["l1_khalf"], HP["l1_pmin"],
                                  HP["l1_taubdt"])
        t.append(time.perf_counter())
        if rewire_period and i % rewire_period == 0 and i // rewire_period < h:
            o.update_mask(st["wmask"], st["weights"], st["Ci"], st["Cj"], st["Cij"], cthr, h, mc,
                          i // rewire_period, 16)
        o.apply_mask(st["weights"], st["wmask"], h, mc)
        t.append(time.perf_counter())
        if timed:
            for name, a, b in zip(split, t[:-1], t[1:]):
                split[name] += b - a
        return xb.shape[0]

    warm_steps = 0
    if warm:  # thread pool, page faults, caches: five steps, fewer when a step takes seconds
        tw = time.perf_counter()
        while warm_steps < 5 and (warm_steps == 0 or time.perf_counter() - tw < 5.0):
            step(warm_steps, False)
            warm_steps += 1
    t0 = time.perf_counter()
    samples = steps = 0
    while steps < min_steps or time.perf_counter() - t0 < budget_s:
        samples += step(1 + steps, True)
        steps += 1
        if steps >= 100000:
            break
    dt = time.perf_counter() - t0
    pool.shutdown()
    limit.restore_original_limits()
    return {"value": samples / dt, "unit": "samples/s", "cores": info["threads_used"], "kind": "port",
            "sample": f"{steps} training step(s) of the same workload (batch {batch}"
                      + (f", rewiring every {rewire_period}th step" if rewire_period else ", no rewiring")
                      + f"), {dt:.1f} s after {warm_steps} warm-up step(s)"
                      + f"; C restatement built -O3 {march} -ffast-math -fopenmp, OMP_PROC_BIND="
                      + os.environ.get("OMP_PROC_BIND", "") + " OMP_PLACES=" + os.environ.get("OMP_PLACES", "")
                      + "; forward through numpy's BLAS kernel, one column slice of W per thread",
            "ms_per_step": 1e3 * dt / max(steps, 1),
            "ms_per_step_by_function": {k: 1e3 * v / max(steps, 1) for k, v in split.items()},
            "host": info}


# ------------------------------------------------------------------------------------------- headline
class DeviceRun:
    def __init__(self, x, y):
        from streambrain_amd import _capi
        self.capi = _capi
        self.lib = _capi.lib()
        _capi.init(0)
        self.net = ctypes.c_void_p()
        _capi.check(self.lib.sb_net_create(ctypes.byref(self.net), 0))
        c = self.capi.check
        c(self.lib.sb_net_add_plastic_layer(self.net, 2 * N_PIXELS, H, MC, HP["l1_taupdt"], HP["l1_pmin"],
                                            HP["l1_khalf"], HP["l1_taubdt"], 1.0, 1.0 / MC, 1.0 / MC))
        c(self.lib.sb_net_add_dense_layer(self.net, H * MC, 1, N_OUT, HP["l2_taupdt"], 1.0 / MC,
                                          1.0 / N_OUT, 1.0 / MC / N_OUT))
        for name, arr in initial_state().items():
            arr = np.ascontiguousarray(arr)
            if name == "wmask":
                self.connected = int(np.count_nonzero(arr))  # rewiring swaps leave this number as it is
            c(self.lib.sb_net_set_layer_state(self.net, 0, name.encode(), arr.ctypes.data, arr.nbytes))
        c(self.lib.sb_net_set_training_data(self.net, x.ctypes.data, y.ctypes.data, x.shape[0], x.shape[1],
                                            y.shape[1]))
        self.ns = x.shape[0]
        self.nb = (self.ns + BATCH - 1) // BATCH
        self.rng = np.random.default_rng(7)

    def close(self):
        self.capi.check(self.lib.sb_net_destroy(self.net))
        self.net = None

    def run_steps(self, first_step, n_steps):
        """Enqueues steps [first_step, first_step + n_steps); returns the number of samples."""
        samples = 0
        for epoch, fb, take in batch_plan(first_step, n_steps, self.nb):
            perm = self.rng.permutation(self.ns).astype(np.int64) if fb == 0 else None
            hc = self.rng.permutation(H).astype(np.int64)
            if fb != 0 and not getattr(self, "_laid_out", False):
                # a run that starts mid-epoch still needs the epoch's sample order applied once
                perm0 = self.rng.permutation(self.ns).astype(np.int64)
                self.capi.check(self.lib.sb_net_train_batches(self.net, 0, BATCH, perm0.ctypes.data,
                                                              hc.ctypes.data, epoch, 0, 0, 0))
            self._laid_out = True
            self.capi.check(self.lib.sb_net_train_batches(
                self.net, 0, BATCH, perm.ctypes.data if perm is not None else None, hc.ctypes.data,
                epoch, fb, take, 0))
            for b in range(fb, fb + take):
                samples += min(BATCH, self.ns - b * BATCH)
        return samples

    def sync(self):
        self.capi.check(self.lib.sb_sync())

    def classifier_steps(self, n_steps):
        """Training steps of the 10-class dense layer (forward of the hidden layer + its fused trace and
        weight update on the labels), batches [0, n_steps) of one epoch; returns the number of samples."""
        n_steps = min(n_steps, self.nb)
        perm = self.rng.permutation(self.ns).astype(np.int64)
        self.capi.check(self.lib.sb_net_train_batches(self.net, 1, BATCH, perm.ctypes.data, None, 0, 0,
                                                      n_steps, 1))
        return sum(min(BATCH, self.ns - b * BATCH) for b in range(n_steps))

    def evaluate(self, x, y):
        correct, total = ctypes.c_int64(0), ctypes.c_int64(0)
        self.capi.check(self.lib.sb_net_evaluate(self.net, x.ctypes.data, y.ctypes.data, x.shape[0],
                                                 x.shape[1], y.shape[1], BATCH, ctypes.byref(correct),
                                                 ctypes.byref(total), None))
        return correct.value, total.value

    def profile(self, first_step, n_steps):
        self.capi.check(self.lib.sb_profile_start())
        self.run_steps(first_step, n_steps)
        self.capi.check(self.lib.sb_profile_stop())
        return read_profile(self.lib, self.capi.check)


def read_profile(lib, check):
    """Per-kernel sums of the HIP events of the last profiled pass: ({name: {launches, raw_avg_us, events}},
    summed event time in ms, number of brackets).  `events`: "carried" when the kernel's launches carry their
    start and stop events themselves (stamped with the dispatch's own begin and end, as a kernel trace reports
    them), "bracket" when the events are recorded on the stream around the launch, which adds to the interval;
    only the latter count as brackets."""
    out, raw_ms, brackets = {}, 0.0, 0
    for k in range(lib.sb_profile_kernels()):
        ms, n = ctypes.c_double(0), ctypes.c_long(0)
        check(lib.sb_profile_get(k, ctypes.byref(ms), ctypes.byref(n)))
        carried = bool(lib.sb_profile_kernel_carried(k))
        raw_ms += ms.value
        brackets += 0 if carried else n.value
        if n.value:
            out[lib.sb_profile_kernel_name(k).decode()] = {"launches": n.value, "raw_avg_us": 1e3 * ms.value / n.value,
                                                           "events": "carried" if carried else "bracket"}
    return out, raw_ms, brackets


def calibrate_brackets(kernels, raw_ms, brackets, unbracketed_s, upper_us=None):
    """A HIP-event bracket adds a little to each launch; how much follows from the two passes themselves:
    (sum of all event intervals - wall time of the same steps without events) / brackets.  Intervals from
    events carried by the launch are the launch's duration as they are."""
    bracket_us = max(0.0, (1e3 * raw_ms - 1e6 * unbracketed_s) / max(brackets, 1))
    # (under a profiler the bracketed pass is slower for reasons of its own: no more than an empty bracket takes)
    if upper_us:
        bracket_us = min(bracket_us, upper_us)
    for k in kernels.values():
        k["avg_us"] = k["raw_avg_us"] if k["events"] == "carried" else max(k["raw_avg_us"] - bracket_us, 0.0)
    return bracket_us


def headline(args):
    x, y = synthetic_dataset(args.samples)
    run = DeviceRun(x, y)
    run.run_steps(0, args.warmup)
    run.sync()
    times, samples_of, first = [], [], args.warmup
    for _ in range(n_windows(args.steps)):
        t0 = time.perf_counter()
        samples_of.append(run.run_steps(first, args.steps))
        run.sync()
        times.append(time.perf_counter() - t0)
        first += args.steps
    mid, windows = window_stats(times, samples_of, args.steps)
    dt, samples = times[mid], samples_of[mid]

    # Per-kernel durations: every launch of one more pass over the same number of steps is bracketed by
    # HIP events on the library's stream.
    # (for a short window the bracketed pass runs on to about 200 steps in one go, so that a 20-step
    # invocation does not price the kernels on 20 launches behind an idle gap)
    n_prof = min(args.steps, 2 * run.nb)
    n_prof *= max(1, min(50, -(-200 // n_prof)))
    prof, raw_ms, brackets = run.profile(first, n_prof)
    bracket_us = calibrate_brackets(prof, raw_ms, brackets, dt * n_prof / args.steps,
                                    run.lib.sb_profile_bracket_overhead_us())

    # the two other phases of the reference's example run, reported beside the headline figure
    # (the first classifier epoch also computes the frozen hidden layer's activations of the whole training
    # set, which later epochs reuse)
    run.sync()
    t1 = time.perf_counter()
    cls_samples = run.classifier_steps(run.nb)
    run.sync()
    cls_first_dt = time.perf_counter() - t1
    t1 = time.perf_counter()
    run.classifier_steps(run.nb)
    run.sync()
    cls_dt = time.perf_counter() - t1
    xt, yt = x[:10000], y[:10000]
    run.evaluate(xt[:BATCH], yt[:BATCH])
    t2 = time.perf_counter()
    run.evaluate(xt, yt)
    ev_dt = time.perf_counter() - t2
    n, m = 2 * N_PIXELS, H * MC
    tw = prof.get("train_fused") or {"avg_us": float("nan")}
    # Algorithmic bytes of the fused training pass: Cij read, Cij written, W written = 12 bytes per synapse
    # (the figure the pass is specified with).  Of these the kernel skips the W entries under zero mask
    # bytes (W stays zero there), so what it has to move at this mask density is less; reported beside.
    connected = run.connected * MC
    alg_bytes = 3 * 4 * n * m
    min_bytes = 2 * 4 * n * m + 4 * connected
    achieved = alg_bytes / (tw["avg_us"] * 1e-6) / 1e9
    # the forward pass multiplies the connected rows of each hypercolumn only
    fwd = prof.get("forward", {"avg_us": float("nan")})
    fwd_flops = 2.0 * BATCH * connected
    fwd_tflops = fwd_flops / (fwd["avg_us"] * 1e-6) / 1e12
    gemm_tflops = 2.0 * BATCH * n * m / (tw["avg_us"] * 1e-6) / 1e12
    traffic, traffic_note = measured_traffic()
    run.close()

    result = {
        "metric": "train samples/sec on 1 MI355X (MNIST-shape fp32 b128); % HBM / MFMA peak",
        "value": samples / dt,
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": 1e3 * dt / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: MNIST-shaped 2-layer network, structural-plasticity layer "
                               "training steps (1568 -> 30x100, mask density 0.1, rewiring every 15th step)",
                   "batch": BATCH, "in_features": n, "hypercolumns": H, "minicolumns": MC,
                   "samples": args.samples},
        "windows": windows,
        "roofline": {"bound": "hbm", "kernel": "k_train_fused", "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_note": traffic_note,
                     "algorithmic_bytes_per_launch": alg_bytes,
                     "bytes_the_kernel_must_move_at_this_mask_density": min_bytes,
                     "avg_launch_us": tw["avg_us"],
                     "trace_gemm_tflops": gemm_tflops, "trace_gemm_frac_of_mfma_peak": gemm_tflops / 157.3},
        "mfma": {"kernel": "k_forward_rows", "flops_per_launch_connected_rows_only": fwd_flops,
                 "achieved_tflops": fwd_tflops, "peak_tflops": 157.3,
                 "frac": fwd_tflops / 157.3, "avg_launch_us": fwd["avg_us"],
                 "trace_gemm_tflops_in_fused_kernel": gemm_tflops},
        "kernels": prof,
        "event_bracket_overhead_us": {"calibrated": bracket_us,
                                      "empty_bracket": run.lib.sb_profile_bracket_overhead_us()},
        "passes": None if args.no_passes else measure_passes(),
        "other_phases": {
            "classifier_layer_train_samples_per_s": cls_samples / cls_dt,
            "classifier_layer_train_first_epoch_samples_per_s": cls_samples / cls_first_dt,
            "evaluate_samples_per_s_host_images_pcie_inclusive": xt.shape[0] / ev_dt,
        },
    }
    if not args.no_cpu_baseline:
        st = initial_state()
        result["cpu_baseline"] = cpu_baseline(x, st, H, MC, BATCH, HP["l1_taupdt"], np.float32,
                                              budget_s=args.cpu_baseline_seconds)
    else:
        result["cpu_baseline"] = None
    if not args.no_other_configs:
        result["other_configs"] = {}
        for name in [w for w in args.other_configs.split(",") if w]:
            steps, warm = SHORT_RUNS[name]
            r = large_workload(name, steps, warm, with_cpu=not args.no_cpu_baseline)
            result["other_configs"][name] = {k: r[k] for k in ("config", "value", "unit", "ms_per_step", "steps",
                                                               "warmup", "windows", "dtype", "roofline", "mfma",
                                                               "cpu_baseline")}
    return result


# Other layer shapes, run through the same network path (one structural-plasticity layer, data resident in
# HBM, first epoch: no rewiring).  in_features, hypercolumns, minicolumns, batch, mask density, dtype,
# samples kept on the device (an epoch of the run cycles through them), fraction of non-zero inputs,
# seconds of CPU baseline (None: not run).
LARGE = {
    "dense": dict(n=1568, h=30, mc=100, batch=128, density=1.0, dtype=np.float32, samples=60000, nonzero=0.19,
                  cpu_s=3.0,
                  what="configs[0]: single hidden layer 1568 -> 30x100, float32, batch 128, dense (no mask), one epoch"),
    "stl10": dict(n=55296, h=200, mc=100, batch=256, density=0.05, dtype=np.float32, samples=5000, nonzero=1.0,
                  cpu_s=0.0,
                  what="configs[3]: STL-10-shaped layer 55296 -> 200x100, float32, batch 256, mask density 0.05"),
    "largest": dict(n=65536, h=1000, mc=100, batch=1024, density=1.0, dtype=np.float32, samples=4096, nonzero=0.2,
                    cpu_s=None,
                    what="configs[4]: 65536 -> 1000x100, float32, batch 1024, binary inputs, dense mask"),
    "mnist15x200": dict(n=1568, h=15, mc=200, batch=128, density=0.1, dtype=np.float32, samples=60000, nonzero=0.19,
                        cpu_s=3.0,
                        what="the reference example script's own MNIST layer: 1568 -> 15x200, float32, batch 128, "
                             "mask density 0.1"),
    "wide64": dict(n=1568, h=100, mc=100, batch=512, density=0.1, dtype=np.float64, samples=60000, nonzero=0.19,
                   cpu_s=3.0,
                   what="configs[2]: 1568 -> 100x100, float64, batch 512, mask density 0.1"),
}
# (timed steps per window, warm-up steps) of the short runs inside the default invocation
SHORT_RUNS = {"dense": (100, 40), "wide64": (40, 20), "stl10": (10, 4), "largest": (3, 2)}


def large_inputs(name):
    cfg = LARGE[name]
    n, ns, dt = cfg["n"], cfg["samples"], cfg["dtype"]
    rng = np.random.default_rng(1000 + len(name))
    if name == "largest":
        x = (rng.random((ns, n), dtype=np.float32) < cfg["nonzero"]).astype(dt)
    else:
        half = n // 2
        px = rng.random((ns, half), dtype=np.float32)
        if cfg["nonzero"] < 1.0:
            px *= rng.random((ns, half), dtype=np.float32) < cfg["nonzero"]
        x = np.concatenate([px, 1.0 - px], axis=1).astype(dt)
    wmask = None
    if cfg["density"] < 1.0:
        wmask = (rng.random((n, cfg["h"]), dtype=np.float32) < cfg["density"]).astype(np.uint8)
    return x, wmask, rng


def large_cpu_baseline(name, x, wmask):
    """CPU baseline of one of the other configurations: same shapes and data, state as the GPU run starts
    from (weights: one block of normal draws repeated, which costs the CPU the same work)."""
    cfg = LARGE[name]
    if cfg["cpu_s"] is None:
        return {"value": None, "unit": "samples/s", "kind": "port",
                "reason": "not run: Cij and W alone need 52 GB of host memory and a step takes minutes "
                          "(about 27 TFLOP of scalar-vector loops per step)"}
    n, h, mc, dt = cfg["n"], cfg["h"], cfg["mc"], cfg["dtype"]
    m = h * mc
    rng = np.random.default_rng(5)
    block = (0.1 * rng.standard_normal(1 << 20)).astype(dt)
    st = {"weights": np.resize(block, (n, m)), "bias": (0.1 * rng.random(m)).astype(dt),
          "Ci": np.ones(n, dtype=dt), "Cj": np.full(m, 1.0 / mc, dtype=dt), "Cij": np.full((n, m), 1.0 / mc, dtype=dt),
          "kbi": np.ones(m, dtype=dt),
          "wmask": wmask if wmask is not None else np.ones((n, h), dtype=np.uint8)}
    st["weights"] = np.ascontiguousarray(st["weights"] * np.repeat(st["wmask"], mc, axis=1).astype(dt)
                                         if wmask is not None and n * m < (1 << 28) else st["weights"])
    tau = HP["l1_taupdt"] * np.sqrt(cfg["batch"] / 128.0)
    big = n * m > (1 << 28)
    return cpu_baseline(x, st, h, mc, cfg["batch"], tau, dt, budget_s=cfg["cpu_s"], min_steps=1,
                        rewire_period=0, warm=not big)


def large_workload(name, steps, warmup, with_cpu=True):
    """Training steps of one structural-plasticity layer of a LARGE shape; returns the result line."""
    from streambrain_amd import _capi
    cfg = LARGE[name]
    n, h, mc, batch, dt = cfg["n"], cfg["h"], cfg["mc"], cfg["batch"], cfg["dtype"]
    m, ns, es = h * mc, cfg["samples"], np.dtype(cfg["dtype"]).itemsize
    x, wmask, rng = large_inputs(name)
    lib = _capi.lib()
    _capi.init(0)
    c = _capi.check
    net = ctypes.c_void_p()
    c(lib.sb_net_create(ctypes.byref(net), 0 if dt == np.float32 else 1))
    tau = HP["l1_taupdt"] * np.sqrt(batch / 128.0)
    c(lib.sb_net_add_plastic_layer(net, n, h, mc, tau, HP["l1_pmin"], HP["l1_khalf"], HP["l1_taubdt"], 1.0,
                                   1.0 / mc, 1.0 / mc))
    # a (never trained) output layer behind it, so that the layer trains on its own activation
    c(lib.sb_net_add_dense_layer(net, m, 1, N_OUT, HP["l2_taupdt"], 1.0 / mc, 1.0 / N_OUT, 1.0 / mc / N_OUT))
    connected = n * h
    if wmask is not None:
        connected = int(np.count_nonzero(wmask))
        c(lib.sb_net_set_layer_state(net, 0, b"wmask", wmask.ctypes.data, wmask.nbytes))
    c(lib.sb_net_set_training_data(net, x.ctypes.data, None, ns, n, 0))
    nb = (ns + batch - 1) // batch

    def run(first, count):
        done = 0
        for epoch, fb, take in batch_plan(first, count, nb):
            perm = rng.permutation(ns).astype(np.int64) if fb == 0 else None
            hc = rng.permutation(h).astype(np.int64)
            c(lib.sb_net_train_batches(net, 0, batch, perm.ctypes.data if perm is not None else None,
                                       hc.ctypes.data, 0, fb, take, 0))
            done += sum(min(batch, ns - b * batch) for b in range(fb, fb + take))
        return done

    warmup = max(warmup, 1)
    run(0, warmup)
    c(lib.sb_sync())
    times, samples_of, first = [], [], warmup
    for _ in range(3):
        t0 = time.perf_counter()
        samples_of.append(run(first, steps))
        c(lib.sb_sync())
        times.append(time.perf_counter() - t0)
        first += steps
    mid, windows = window_stats(times, samples_of, steps)
    dt_s, samples = times[mid], samples_of[mid]
    c(lib.sb_profile_start())
    n_prof = min(steps, nb)
    run(first, n_prof)
    c(lib.sb_profile_stop())
    kernels, raw_ms, brackets = read_profile(lib, c)
    bracket_us = calibrate_brackets(kernels, raw_ms, brackets, dt_s * n_prof / steps,
                                    lib.sb_profile_bracket_overhead_us())
    c(lib.sb_net_destroy(net))
    tw = kernels.get("train_fused", {"avg_us": float("nan")})["avg_us"] * 1e-6
    fw = kernels.get("forward", {"avg_us": float("nan")})["avg_us"] * 1e-6
    dname = "f32" if dt == np.float32 else "f64"
    peak = MFMA_PEAK_TFLOPS[dname]
    gemm = 2.0 * batch * n * m  # the Cij trace GEMM of a full batch
    fwd_flops = 2.0 * batch * connected * mc if cfg["density"] <= 0.5 else gemm
    stream_bytes = 3 * es * n * m
    # which roof bounds the fused kernel: its GEMM at the MFMA peak against its 3 s N M stream at the HBM peak
    mfma_bound = gemm / (peak * 1e12) >= stream_bytes / (HBM_PEAK_GBS * 1e9)
    if mfma_bound:
        roofline = {"bound": "mfma", "kernel": "k_train_fused", "achieved": gemm / tw / 1e12, "peak": peak,
                    "unit": "TFLOP/s", "frac": gemm / tw / 1e12 / peak, "traffic": None,
                    "algorithmic_flops_per_launch": gemm, "avg_launch_us": tw * 1e6,
                    "bytes_3sNM_per_launch": stream_bytes, "achieved_GBps_on_3sNM": stream_bytes / tw / 1e9}
    else:
        roofline = {"bound": "hbm", "kernel": "k_train_fused", "achieved": stream_bytes / tw / 1e9,
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": stream_bytes / tw / 1e9 / HBM_PEAK_GBS,
                    "traffic": None, "algorithmic_bytes_per_launch": stream_bytes, "avg_launch_us": tw * 1e6,
                    "trace_gemm_tflops": gemm / tw / 1e12, "trace_gemm_frac_of_mfma_peak": gemm / tw / 1e12 / peak}
    return {
        "metric": "train samples/sec on 1 MI355X; % HBM / MFMA peak",
        "value": samples / dt_s, "unit": "samples/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": 1e3 * dt_s / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic",
        "config": {"workload": cfg["what"], "batch": batch, "in_features": n, "hypercolumns": h,
                   "minicolumns": mc, "samples": ns},
        "windows": windows,
        "roofline": roofline,
        "mfma": {"kernel": "k_forward_rows" if cfg["density"] <= 0.5 else "k_forward",
                 "flops_per_launch": fwd_flops, "achieved_tflops": fwd_flops / fw / 1e12, "peak_tflops": peak,
                 "frac": fwd_flops / fw / 1e12 / peak, "avg_launch_us": fw * 1e6},
        "kernels": kernels, "event_bracket_overhead_us": {"calibrated": bracket_us},
        "cpu_baseline": large_cpu_baseline(name, x, wmask) if with_cpu else None}


# ------------------------------------------------------------------------- counters, peaks, summaries
def kernel_source_stamp():
    """sha256 over the sources of the dominant kernel: a counter summary in profiles/ names the stamp of
    the sources it was measured with."""
    hsh = hashlib.sha256()
    for f in KERNEL_SOURCES:
        hsh.update(open(os.path.join(ROOT, "streambrain_amd", "csrc", f), "rb").read())
    return hsh.hexdigest()[:16]


def measured_traffic():
    """HBM bytes per launch of the dominant kernel, as measured with rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE and recorded in profiles/ (lines `traffic_bytes_per_launch: N`, `kernel_source_stamp: S`);
    (None, why) when there is no summary or it was measured with other kernel sources."""
    traffic = stamp = None
    try:
        for line in open(PMC_PROFILE):
            if line.startswith("traffic_bytes_per_launch:"):
                traffic = float(line.split(":", 1)[1])
            if line.startswith("kernel_source_stamp:"):
                stamp = line.split(":", 1)[1].strip()
    except OSError:
        return None, "no counter summary in profiles/"
    if traffic is None:
        return None, "no traffic line in the counter summary"
    if stamp != kernel_source_stamp():
        return None, "the counter summary in profiles/ was measured with other kernel sources"
    return traffic, "rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a plain copy (profiles/)"


def copy_calibration(nbytes=64 << 20, copies=6):
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray
    _capi.init(0)
    lib = _capi.lib()
    src, dst = DeviceArray((nbytes,), np.uint8), DeviceArray((nbytes,), np.uint8)
    _capi.check(lib.sb_fill_bytes(src.ptr, 1, nbytes))
    _capi.check(lib.sb_fill_bytes(dst.ptr, 2, nbytes))
    for _ in range(copies):
        _capi.check(lib.sb_memcpy_d2d(dst.ptr, src.ptr, nbytes))
    _capi.check(lib.sb_sync())
    print(json.dumps({"copy_calibration": {"copies": copies, "bytes_read_per_copy": nbytes,
                                           "bytes_written_per_copy": nbytes}}))
    return 0


def achievable_peaks():
    """What the box reaches in practice, next to the published peaks: device-to-device copies of three
    sizes (bytes read + written per second) and MFMA-only kernels in float and double."""
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray
    _capi.init(0)
    lib, c = _capi.lib(), _capi.check
    out = {"hbm_peak_GBps_published": HBM_PEAK_GBS, "copies": [], "mfma": []}
    for nbytes in (32 << 20, 128 << 20, 2 << 30):
        src, dst = DeviceArray((nbytes,), np.uint8), DeviceArray((nbytes,), np.uint8)
        c(lib.sb_fill_bytes(src.ptr, 1, nbytes))
        c(lib.sb_fill_bytes(dst.ptr, 2, nbytes))
        reps = max(4, min(200, (8 << 30) // nbytes))
        best = float("inf")
        for _ in range(3):
            c(lib.sb_sync())
            t0 = time.perf_counter()
            for _ in range(reps):
                c(lib.sb_memcpy_d2d(dst.ptr, src.ptr, nbytes))
            c(lib.sb_sync())
            best = min(best, (time.perf_counter() - t0) / reps)
        out["copies"].append({"bytes": nbytes, "copies_timed": reps, "us_per_copy": 1e6 * best,
                              "GBps_read_plus_written": 2 * nbytes / best / 1e9,
                              "frac_of_published_peak": 2 * nbytes / best / 1e9 / HBM_PEAK_GBS})
        src.free()
        dst.free()
    for dtype, name, shape in ((0, "f32", "16x16x4"), (1, "f64", "16x16x4"), (2, "f64", "4x4x4 (four blocks)")):
        flops = ctypes.c_double(0)
        c(lib.sb_probe_mfma(dtype, 2048, 1000, ctypes.byref(flops)))  # warm-up
        c(lib.sb_sync())
        for iters, what in ((1000, "short launch (a few ms)"), (20000, "long launch (tens of ms)")):
            best = float("inf")
            for _ in range(3):
                t0 = time.perf_counter()
                c(lib.sb_probe_mfma(dtype, 2048, iters, ctypes.byref(flops)))
                c(lib.sb_sync())
                best = min(best, time.perf_counter() - t0)
            out["mfma"].append({"dtype": name, "instruction": shape, "workgroups": 2048, "what": what,
                                "flops": flops.value, "ms": 1e3 * best, "TFLOPps": flops.value / best / 1e12,
                                "published_peak_TFLOPps": MFMA_PEAK_TFLOPS[name],
                                "frac_of_published_peak": flops.value / best / 1e12 / MFMA_PEAK_TFLOPS[name]})
    print(json.dumps({"achievable_peaks": out}))
    return 0


def entry_point_rates(reps=200):
    """The per-function entry points of the C ABI on device buffers at the headline layer's shape
    (1568 -> 30 x 100, batch 128, mask density 0.1), each launched `reps` times back to back: time per
    call and the rate on its algorithmic bytes or flops.  The network path uses the fused kernels; these
    are what a caller that drives the reference's functions one by one gets."""
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray
    _capi.init(0)
    lib, c = _capi.lib(), _capi.check
    n, h, mc, b = 1568, 30, 100, 128
    m = h * mc
    rows = []
    for dtype, sfx, R in ((np.float32, "_f32", ctypes.c_float), (np.float64, "_f64", ctypes.c_double)):
        rng = np.random.default_rng(0)
        es = np.dtype(dtype).itemsize
        x = DeviceArray.from_numpy(rng.random((b, n)).astype(dtype))
        act = DeviceArray.from_numpy(rng.random((b, m)).astype(dtype))
        W = DeviceArray.from_numpy((0.1 * rng.standard_normal((n, m))).astype(dtype))
        bias = DeviceArray.from_numpy(rng.random(m).astype(dtype))
        kbi = DeviceArray.from_numpy(np.ones(m, dtype))
        Ci = DeviceArray.from_numpy((0.05 + 0.1 * rng.random(n)).astype(dtype))
        Cj = DeviceArray.from_numpy((0.005 + 0.01 * rng.random(m)).astype(dtype))
        Cij = DeviceArray.from_numpy((0.001 * rng.random((n, m))).astype(dtype))
        mask_host = (rng.random((n, h)) < 0.1).astype(np.uint8)
        wmask = DeviceArray.from_numpy(mask_host)
        pred = DeviceArray((b,), np.int32)
        tau, cthr = 0.0001, 0.00005
        masked_bytes = int((mask_host == 0).sum()) * mc * es + n * h
        calls = [
            ("sb_update_state", lambda: getattr(lib, "sb_update_state" + sfx)(act.ptr, x.ptr, W.ptr, bias.ptr, b, n, m),
             None, 2.0 * b * n * m),
            ("sb_softmax_minicolumns", lambda: getattr(lib, "sb_softmax_minicolumns" + sfx)(act.ptr, b, h, mc),
             2 * b * m * es, None),
            ("sb_compute_activation", lambda: getattr(lib, "sb_compute_activation" + sfx)(act.ptr, x.ptr, W.ptr, bias.ptr, b, n,
                                                                               h, mc), None, 2.0 * b * n * m),
            ("sb_add_bias", lambda: getattr(lib, "sb_add_bias" + sfx)(act.ptr, bias.ptr, b, m), 2 * b * m * es, None),
            ("sb_update_weights", lambda: getattr(lib, "sb_update_weights" + sfx)(Ci.ptr, Cj.ptr, Cij.ptr, x.ptr, act.ptr,
                                                                        R(tau), W.ptr, R(cthr), b, n, m),
             3 * n * m * es, 2.0 * b * n * m),
            ("sb_update_counters", lambda: getattr(lib, "sb_update_counters" + sfx)(Ci.ptr, Cj.ptr, Cij.ptr, x.ptr, act.ptr,
                                                                          R(tau), b, n, m),
             2 * n * m * es, 2.0 * b * n * m),
            ("sb_weights_from_counters", lambda: getattr(lib, "sb_weights_from_counters" + sfx)(W.ptr, Ci.ptr, Cj.ptr, Cij.ptr,
                                                                                      R(cthr), n, m),
             2 * n * m * es, None),
            ("sb_apply_mask", lambda: getattr(lib, "sb_apply_mask" + sfx)(W.ptr, wmask.ptr, n, h, mc), masked_bytes, None),
            ("sb_update_bias_regularized",
             lambda: getattr(lib, "sb_update_bias_regularized" + sfx)(bias.ptr, kbi.ptr, Cj.ptr, R(cthr), R(-500.0), R(0.3),
                                                            R(0.0002), m), 4 * m * es, None),
            ("sb_argmax_rows", lambda: getattr(lib, "sb_argmax_rows" + sfx)(act.ptr, b, m, pred.ptr), b * m * es, None),
        ]
        for name, call, nbytes, flops in calls:
            for _ in range(10):
                c(call())
            best = float("inf")
            for _ in range(3):
                c(lib.sb_sync())
                t0 = time.perf_counter()
                for _ in range(reps):
                    c(call())
                c(lib.sb_sync())
                best = min(best, (time.perf_counter() - t0) / reps)
            row = {"entry_point": name + sfx, "us_per_call": round(1e6 * best, 2), "calls_timed": reps}
            if nbytes is not None:
                row["algorithmic_bytes"] = nbytes
                row["GBps"] = round(nbytes / best / 1e9, 1)
                row["frac_of_hbm_peak"] = round(nbytes / best / 1e9 / HBM_PEAK_GBS, 3)
            if flops is not None:
                peak = MFMA_PEAK_TFLOPS["f32" if es == 4 else "f64"]
                row["flops"] = flops
                row["TFLOPps"] = round(flops / best / 1e12, 2)
                row["frac_of_mfma_peak"] = round(flops / best / 1e12 / peak, 3)
            rows.append(row)
        for d in (x, act, W, bias, kbi, Ci, Cj, Cij, wmask, pred):
            d.free()
    print(json.dumps({"entry_point_rates": {"shape": {"N": n, "H": h, "Mc": mc, "batch": b, "mask_density": 0.1},
                                            "note": "back-to-back launches on the library's stream; a call of a few "
                                                    "microseconds is bound by launch and completion (about 2.7 us)",
                                            "rows": rows}}))
    return 0


def measure_passes(reps=300):
    """The passes of the training step one by one at the headline layer's shape (1568 -> 30 x 100, float32,
    batch 128, mask density 0.1), each through its own C entry point on device buffers, `reps` launches back
    to back, timed twice: wall clock per call without brackets, and with every launch bracketed by HIP
    events on the library's stream (the headline's per-kernel brackets).  For the passes that are one launch
    per call the first is the launch's duration, and their difference is what a bracket adds; the trace pass's
    entry point is two launches (the training kernel, then the copy of the new Ci / Cj over the caller's), so
    its kernel is priced from its brackets minus that difference:
      trace pass     Ci/Cj/Cij moving averages, the Cij one as the MFMA GEMM x^T y with the decay in its
                     epilogue (sb_update_counters: the fused training kernel without the weights)
      weight pass    W = log(max(Cij, cthr^4) / (Ci Cj)) streamed over Cij (sb_weights_from_counters), and
                     the same with the mask apply fused in (sb_weights_masked_from_counters)
      forward        the dense x.W + bias GEMM with the softmax epilogue (sb_compute_activation)
    Rates are on the algorithmic bytes / flops of each pass, against the published peaks."""
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray
    _capi.init(0)
    lib, c = _capi.lib(), _capi.check
    n, h, mc, b, es = 2 * N_PIXELS, H, MC, BATCH, 4
    m = h * mc
    rng = np.random.default_rng(0)
    f = np.float32
    x = DeviceArray.from_numpy((rng.random((b, n)) * (rng.random((b, n)) < 0.6)).astype(f))
    act = DeviceArray.from_numpy(numpy_softmax(rng.standard_normal((b, m)), h, mc).astype(f))
    out = DeviceArray((b, m), f)
    W = DeviceArray.from_numpy((0.1 * rng.standard_normal((n, m))).astype(f))
    bias = DeviceArray.from_numpy((0.1 * rng.random(m)).astype(f))
    Ci = DeviceArray.from_numpy((0.3 + 0.1 * rng.random(n)).astype(f))
    Cj = DeviceArray.from_numpy((0.005 + 0.01 * rng.random(m)).astype(f))
    Cij = DeviceArray.from_numpy((0.003 * (0.1 + rng.random((n, m)))).astype(f))
    mask_host = (rng.random((n, h)) < HP["l1_density"]).astype(np.uint8)
    wmask = DeviceArray.from_numpy(mask_host)
    connected = int(mask_host.sum()) * mc
    tau, cthr = HP["l1_taupdt"], HP["l1_taupdt"] / 2
    R = ctypes.c_float
    calls = {
        "trace": (lambda: lib.sb_update_counters_f32(Ci.ptr, Cj.ptr, Cij.ptr, x.ptr, act.ptr, R(tau), b, n, m),
                  "train_fused"),
        "weight": (lambda: lib.sb_weights_from_counters_f32(W.ptr, Ci.ptr, Cj.ptr, Cij.ptr, R(cthr), n, m),
                   "weight_pass"),
        "weight_masked": (lambda: lib.sb_weights_masked_from_counters_f32(W.ptr, Ci.ptr, Cj.ptr, Cij.ptr, wmask.ptr,
                                                                          R(cthr), n, h, mc), "weight_pass"),
        "forward_dense": (lambda: lib.sb_compute_activation_f32(out.ptr, x.ptr, W.ptr, bias.ptr, b, n, h, mc),
                          "forward"),
    }
    measured = {}
    for name, (call, kernel) in calls.items():
        for _ in range(20):
            c(call())
        c(lib.sb_sync())
        t0 = time.perf_counter()
        for _ in range(reps):
            c(call())
        c(lib.sb_sync())
        wall_us = 1e6 * (time.perf_counter() - t0) / reps
        c(lib.sb_profile_start())
        for _ in range(reps):
            c(call())
        c(lib.sb_profile_stop())
        prof, _, _ = read_profile(lib, c)
        measured[name] = {"launches": prof[kernel]["launches"], "raw_avg_us": prof[kernel]["raw_avg_us"],
                          "events": prof[kernel]["events"], "wall_us_per_call_back_to_back": wall_us}
    singles = sorted(measured[k]["raw_avg_us"] - measured[k]["wall_us_per_call_back_to_back"]
                     for k in ("weight", "weight_masked", "forward_dense"))
    bracket_us = max(singles[1], 0.0)
    for name, v in measured.items():
        if name == "trace":
            v["avg_us"] = v["raw_avg_us"] if v["events"] == "carried" else v["raw_avg_us"] - bracket_us
        else:
            v["avg_us"] = v["wall_us_per_call_back_to_back"]
    gemm = 2.0 * b * n * m
    peak = MFMA_PEAK_TFLOPS["f32"]

    def hbm(t_us, nbytes):
        return {"algorithmic_bytes": nbytes, "GBps": nbytes / (t_us * 1e-6) / 1e9,
                "frac_of_hbm_peak": nbytes / (t_us * 1e-6) / 1e9 / HBM_PEAK_GBS}

    def mfma(t_us, flops):
        return {"flops": flops, "TFLOPps": flops / (t_us * 1e-6) / 1e12,
                "frac_of_mfma_peak": flops / (t_us * 1e-6) / 1e12 / peak}

    t = {k: v["avg_us"] for k, v in measured.items()}
    passes = {
        "shape": {"in_features": n, "hypercolumns": h, "minicolumns": mc, "batch": b, "mask_density": HP["l1_density"],
                  "dtype": "f32"},
        "how": f"{reps} calls back to back per pass; avg_us = wall clock per call for the one-launch passes; for "
               "the trace pass the kernel's own duration from events its launch carries (the call has a second, "
               "small launch)",
        "event_bracket_overhead_us": bracket_us,
        "trace": dict(measured["trace"], kernel="k_train_fused, traces only (sb_update_counters; the Ci / Cj copy "
                                                "back of that entry point is a separate launch, not timed here)",
                      mfma=mfma(t["trace"], gemm), hbm=hbm(t["trace"], 2 * es * n * m + es * b * (n + m))),
        "weight": dict(measured["weight"], kernel="k_weight_pass, no mask (sb_weights_from_counters)",
                       hbm=hbm(t["weight"], 2 * es * n * m)),
        "weight_masked": dict(measured["weight_masked"],
                              kernel="k_weight_pass with the mask apply (sb_weights_masked_from_counters)",
                              hbm=hbm(t["weight_masked"], 2 * es * n * m + n * h),
                              bytes_the_kernel_must_move_at_this_mask_density=es * n * m + es * connected + n * h),
        "forward_dense": dict(measured["forward_dense"], kernel="k_forward (sb_compute_activation, dense W)",
                              mfma=mfma(t["forward_dense"], gemm)),
    }
    for d in (x, act, out, W, bias, Ci, Cj, Cij, wmask):
        d.free()
    return passes


def _pmc_medians(directory):
    import collections
    import csv
    import glob
    import re
    files = []
    for d in directory.split(","):  # several runs' directories, comma-separated
        files += sorted(glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True))
    res = collections.defaultdict(lambda: collections.defaultdict(list))
    for f in files:
        for row in csv.DictReader(open(f)):
            k = re.sub(r"^void sb::", "", re.sub(r"\(.*", "", row["Kernel_Name"]))
            res[k][row["Counter_Name"]].append(float(row["Counter_Value"]))
    return {k: {c: (len(v), sorted(v)[len(v) // 2]) for c, v in d.items()} for k, d in res.items()}


def trace_summary(directory):
    """Per-kernel table (calls, average / minimum / maximum duration, share of GPU time) from the
    *_kernel_stats.csv files that `rocprofv3 --kernel-trace --stats --output-format csv` wrote below
    `directory`."""
    import csv
    import glob
    import re
    for f in sorted(glob.glob(os.path.join(directory, "**", "*kernel_stats.csv"), recursive=True)):
        print(f"{'kernel':62s} {'calls':>7s} {'avg us':>9s} {'min us':>9s} {'max us':>9s} {'% of GPU time':>14s}")
        for r in csv.DictReader(open(f)):
            name = re.sub(r"^void sb::", "", re.sub(r"\(.*", "", r["Name"]))[:62]
            print(f"{name:62s} {int(r['Calls']):7d} {float(r['AverageNs']) / 1e3:9.2f} {float(r['MinNs']) / 1e3:9.2f} "
                  f"{float(r['MaxNs']) / 1e3:9.2f} {float(r['Percentage']):14.2f}")
    return 0


def pmc_summary(directory, calibration=None):
    """Per-kernel medians of the counters in the rocprofv3 --pmc output below `directory` (csv format) as
    text.  With `calibration` (the output of the same counters over `bench.py --copy-calibration`),
    FETCH_SIZE / WRITE_SIZE (KiB per dispatch) are scaled by what they read for the plain 64 MiB copies and
    the traffic of the fused training kernel is printed as the line bench.py reads back."""
    med = _pmc_medians(directory)
    print(f"kernel_source_stamp: {kernel_source_stamp()}")
    scale = {}
    if calibration:
        cal = _pmc_medians(calibration)
        copy = next((d for k, d in cal.items() if "copyBuffer" in k or "copy" in k.lower()), None)
        if copy:
            for cname in ("FETCH_SIZE", "WRITE_SIZE"):
                if cname in copy and copy[cname][1] > 0:
                    scale[cname] = 65536.0 / copy[cname][1]
                    print(f"calibration: plain device copy of 64 MiB reads {cname} = {copy[cname][1]:.1f} KiB "
                          f"-> scale {scale[cname]:.4f}")
    for k, d in sorted(med.items()):
        print(k)
        for cname, (n, v) in sorted(d.items()):
            extra = f"  = {v * 1024 * scale[cname] / 1e6:10.2f} MB per launch" if cname in scale else ""
            print(f"   {cname:32s} launches={n:5d} median={v:16.1f}{extra}")
    fused = [d for k, d in med.items() if k.startswith("k_train_fused")]
    if fused and len(scale) == 2 and all(c in fused[0] for c in scale):
        total = sum(fused[0][c][1] * 1024 * scale[c] for c in scale)
        print(f"traffic_bytes_per_launch: {total:.0f}")
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=938)
    ap.add_argument("--warmup", type=int, default=60)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="leave out the short runs of the other four configurations")
    ap.add_argument("--other-configs", default="dense,wide64,stl10,largest",
                    help="which of the other configurations the default run adds (comma-separated)")
    ap.add_argument("--cpu-baseline-seconds", type=float, default=15.0,
                    help="length of the headline CPU baseline's sample")
    ap.add_argument("--samples", type=int, default=N_SAMPLES)
    ap.add_argument("--workload", choices=["mnist"] + sorted(LARGE), default="mnist",
                    help="mnist (default): the headline configuration with short runs of the others; the "
                         "others: one layer of that shape alone (--steps defaults to two epochs of its "
                         "resident samples)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run six 64 MiB device-to-device copies: the known-size kernel that "
                         "hardware counter readings (FETCH_SIZE, WRITE_SIZE) are scaled by")
    ap.add_argument("--achievable-peaks", action="store_true",
                    help="only measure device-copy bandwidth and MFMA-only kernels (what the box reaches "
                         "next to the published peaks)")
    ap.add_argument("--entry-point-rates", action="store_true",
                    help="only time the per-function entry points of the C ABI at the headline layer's shape")
    ap.add_argument("--no-passes", action="store_true",
                    help="leave the passes one by one out of the default run (a kernel trace of the run then holds "
                         "the pipeline's launches only)")
    ap.add_argument("--passes", action="store_true",
                    help="only time the passes of the training step one by one (trace, weight, forward) at the "
                         "headline layer's shape")
    ap.add_argument("--trace-summary", metavar="DIR",
                    help="per-kernel table from rocprofv3 --kernel-trace --stats csv output below DIR")
    ap.add_argument("--pmc-summary", metavar="DIR", help="summarise rocprofv3 --pmc csv output below DIR")
    ap.add_argument("--pmc-calibration", metavar="DIR",
                    help="with --pmc-summary: the same counters over `bench.py --copy-calibration`")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              "(the path is not sharded across devices)", file=sys.stderr)
        return 2
    if args.trace_summary:
        return trace_summary(args.trace_summary)
    if args.pmc_summary:
        return pmc_summary(args.pmc_summary, args.pmc_calibration)
    if args.copy_calibration:
        return copy_calibration()
    if args.achievable_peaks:
        return achievable_peaks()
    if args.entry_point_rates:
        return entry_point_rates()
    if args.passes:
        print(json.dumps({"passes": measure_passes()}))
        return 0
    if args.workload != "mnist":
        cfg = LARGE[args.workload]
        nb = (cfg["samples"] + cfg["batch"] - 1) // cfg["batch"]
        steps = args.steps if "--steps" in sys.argv else (nb if nb > 100 else 2 * nb)
        print(json.dumps(large_workload(args.workload, steps, args.warmup if "--warmup" in sys.argv else nb,
                                        with_cpu=not args.no_cpu_baseline)))
        return 0
    print(json.dumps(headline(args)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
