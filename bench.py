"""Benchmark of the signature hot path on one MI355X.

A "step" is one forward + one backward pass of the headline workload
(batch 32, length 1000, dimension 10, degree 5, float64; path points iid N(0,1))
through the library's C ABI with all buffers resident in HBM.  Prints ONE JSON line.

Order of a run: every other leg first (configs 2-4, the extra shapes, stream-ordered mode, per-kernel timings), then the
headline: W untimed warm-up steps, K timed steps, each step timed on its own (both calls are synchronous); after it the
same calls through the Python wrappers and the measured FMA ceilings.
`ms_per_step` is the median step, `ms_per_step_mean` the mean over the same K steps; `value` follows the median.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--all-configs]
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"float64": 78.6, "float32": 157.3}

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "sweep_kernels_hbm_traffic.txt")


def traffic_bytes(instance):
    """HBM bytes per launch of a sweep kernel as measured with rocprofv3 (FETCH_SIZE / WRITE_SIZE scaled by a plain copy
    of known size), read from the committed summary; None when the summary has no row for this instance, e.g. after a
    partition was re-tuned.  `instance` is the library's name, e.g. bwd_f64_d10_n5_t2_k5_lds[_ll]."""
    import re
    m = re.match(r"^(fwd|bwd)_(f64|f32)_d(\d+)_n(\d+)_t(\d+)_k(\d+)(_lds)?(_ll)?$", instance)
    if not m or not os.path.exists(TRAFFIC_PROFILE):
        return None
    d = int(m.group(3))
    ll = 0 if not m.group(8) else (1 if d % 2 else 2)
    row = "tree_%s_kernel<%s, %d, %s, %s, %s, %s, %d>" % (m.group(1), "double" if m.group(2) == "f64" else "float", d, m.group(4),
                                                           m.group(5), m.group(6), "true" if m.group(7) else "false", ll)
    with open(TRAFFIC_PROFILE) as fh:
        for line in fh:
            if line.startswith(row):
                cols = line[len(row):].split()
                if len(cols) >= 3:
                    return float(cols[2]) * 1e6      # columns: FETCH KiB, WRITE KiB, traffic MB, algorithmic MB
    return None


def measured_peaks(loader):
    """Independent FMAs and nothing else, at 1 / 2 / 8 waves per SIMD (a kernel of the library): the ceiling the chip
    reaches against the nominal peak.  The headline sweeps run one wave per SIMD."""
    fn = loader.CUSIG.cusig_amd_measure_fma_peak
    fn.argtypes = (ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double))
    fn.restype = ctypes.c_int
    out = {}
    for name, is_f64 in (("f64", 1), ("f32_unpacked", 0)):
        out[name] = {}
        for waves in (1, 2, 8):
            v = ctypes.c_double()
            rc = fn(is_f64, waves, ctypes.byref(v))
            out[name]["%d_waves_per_simd" % waves] = v.value if rc == 0 else None
    return out


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step is about 1 ms: the defaults run long enough for the GPU clocks to settle under load
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--all-configs", action="store_true", help="(default) also time configs 2-4, reported under 'configs'")
    ap.add_argument("--headline-only", action="store_true", help="time only the headline workload (configs 1 and 5)")
    ap.add_argument("--ops", action="store_true",
                    help="time the operators either side of the sweep (sig_combine, sig_join, linear_sig, transform_path "
                         "and backward passes) on HBM-bound shapes and print their own JSON line instead")
    ap.add_argument("--copy-calib", action="store_true",
                    help="only run a plain 256 MiB device copy (calibrates rocprofv3 FETCH_SIZE / WRITE_SIZE) and exit")
    return ap.parse_args()


class Runner:
    """Holds device buffers of one config and calls the C ABI on raw pointers."""

    def __init__(self, k, torch, np, loader, cfgmod):
        c = cfgmod.CONFIGS[k]
        self.k, self.c = k, c
        self.torch, self.loader = torch, loader
        self.np_path = cfgmod.make_path(k)
        self.d_aug = cfgmod.aug_dim(c)
        self.L = cfgmod.n_increments(c)
        self.dtype = c["dtype"]
        tdt = torch.float64 if self.dtype == "float64" else torch.float32
        self.path = torch.tensor(self.np_path, device="cuda:0")
        n = int(loader.CUSIG.cusig_amd_sig_length(self.d_aug, c["degree"])) - 1
        self.sig = torch.empty((c["batch"], n), dtype=tdt, device="cuda:0")
        self.real = loader.DTYPES[self.dtype]
        self.flops_fwd = c["batch"] * self.L * cfgmod.flops_fwd(self.d_aug, c["degree"])
        self.flops_bwd = c["batch"] * self.L * cfgmod.flops_bwd(self.d_aug, c["degree"])
        self.grad = None
        self.gsig = None
        if c["backward"]:
            rng = np.random.default_rng(2000 + k)
            self.gsig = torch.tensor(rng.standard_normal((c["batch"], n)).astype(self.dtype), device="cuda:0")
            self.grad = torch.empty_like(self.path)
        # the argument lists are built once: a call is then one ctypes call
        self._fwd = loader.CUSIG_SIGNATURE[self.dtype]
        self._fwd_args = (self._p(self.path), self._p(self.sig), c["batch"], c["dim"], c["length"], c["degree"], c["time_aug"],
                          c["lead_lag"], 1.0, True, False, None, 0, 0, 0)
        if c["backward"]:
            self._bwd = loader.CUSIG_SIG_BACKPROP[self.dtype]
            self._bwd_args = (self._p(self.path), self._p(self.grad), self._p(self.gsig), self._p(self.sig), c["batch"], c["dim"],
                              c["length"], c["degree"], c["time_aug"], c["lead_lag"], 1.0, False, None, 0, 0, 0)

    def _p(self, t):
        return ctypes.cast(t.data_ptr(), ctypes.POINTER(self.real))

    def forward(self):
        rc = self._fwd(*self._fwd_args)
        if rc:
            raise RuntimeError("signature_cuda failed: %d %s" % (rc, self.loader.last_error_message()))

    def backward(self):
        rc = self._bwd(*self._bwd_args)
        if rc:
            raise RuntimeError("sig_backprop_cuda failed: %d %s" % (rc, self.loader.last_error_message()))


def time_calls(fn, torch, loader, warmup, steps):
    """Returns (median wall seconds per call, mean sweep-kernel ms, kernel name)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    loader.CUSIG.cusig_amd_set_profiling(1)
    kms, walls = [], []
    for _ in range(steps):
        t0 = time.perf_counter()
        fn()
        walls.append(time.perf_counter() - t0)
        kms.append(float(loader.CUSIG.cusig_amd_last_kernel_ms()))
    torch.cuda.synchronize()
    name = loader.CUSIG.cusig_amd_last_kernel_name().decode()
    loader.CUSIG.cusig_amd_set_profiling(0)
    return statistics.median(walls), sum(kms) / len(kms), name


def time_steps(step, torch, warmup, steps):
    """W untimed warm-up steps, then K steps timed one by one between two device synchronisations.
    Returns (median ms, mean ms)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t_all = time.perf_counter()
    each = []
    for _ in range(steps):
        t0 = time.perf_counter()
        step()
        each.append(time.perf_counter() - t0)
    torch.cuda.synchronize()
    mean_ms = (time.perf_counter() - t_all) / steps * 1e3
    return statistics.median(each) * 1e3, mean_ms


def cpu_model():
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(np, cfgmod):
    """The CPU oracle (restatement of the reference's cpsig algorithm) on all host threads, same workload."""
    from oracle import sigref
    x = cfgmod.make_path(1)
    c = cfgmod.CONFIGS[1]
    # one path per thread (the reference's chunking): at most `batch` threads do work.  A process that is given a
    # CPU share smaller than the machine (OMP_NUM_THREADS says so) uses that share.
    threads = min(sigref.max_threads(), c["batch"])
    share = os.environ.get("OMP_NUM_THREADS", "")
    if share.isdigit() and int(share) > 0:
        threads = min(threads, int(share))
    rng = np.random.default_rng(2005)
    best = None
    sig = None
    g = None
    reps = 60       # about 0.13 s each on 16 host threads: ~8 s of CPU work
    for _ in range(reps):
        t0 = time.perf_counter()
        sig = sigref.signature(x, c["degree"], n_jobs=threads)
        t1 = time.perf_counter()
        if g is None:
            g = rng.standard_normal(sig.shape)
        t2 = time.perf_counter()
        sigref.sig_backprop(x, sig, g, c["degree"], n_jobs=threads)
        t3 = time.perf_counter()
        dt = (t1 - t0) + (t3 - t2)
        best = dt if best is None else min(best, dt)
    return {"value": c["batch"] / best, "unit": "signatures/s (fwd+bwd)", "cores": threads, "kind": "port",
            "os_cpu_count": os.cpu_count(), "hardware_threads": sigref.max_threads(), "cpu_model": cpu_model(),
            "sample": "full headline workload (32 paths x 999 steps, d=10, degree 5, f64), best of %d, "
                      "oracle/sigref.c -O3 -march=native, one path per thread on %d threads (the process's CPU share)"
                      % (reps, threads)}


def bench_ops(args, torch, loader):
    """Operators either side of the sweep: HBM-bound element-wise kernels.  Achieved GB/s = algorithmic bytes (every
    input read once, every output written once) / wall time of the synchronous C-ABI call."""
    real = loader.DTYPES["float64"]
    d, deg, batch = 10, 5, 1024
    n = int(loader.CUSIG.cusig_amd_sig_length(d, deg)) - 1
    f64 = dict(dtype=torch.float64, device="cuda:0")
    a = torch.rand((batch, n), **f64) * 0.1
    b = torch.rand((batch, n), **f64) * 0.1
    g = torch.rand((batch, n), **f64)
    z = torch.rand((batch, d), **f64)
    o1, o2, oz = torch.empty_like(a), torch.empty_like(a), torch.empty_like(z)
    pb, plen, pdim = 4096, 1024, 16
    path = torch.rand((pb, plen, pdim), **f64)
    tpath = torch.empty((pb, 2 * plen - 1, 2 * pdim + 1), **f64)
    gpath = torch.empty_like(path)

    def p(t):
        return ctypes.cast(t.data_ptr(), ctypes.POINTER(real))

    def pu(t):
        return ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_uint64))

    # sig_coef: every word of 3 letters over 10 channels (1000 words, prefixes layout), 256 paths of 1000 points
    import itertools
    words = list(itertools.product(range(d), repeat=3))
    n_words, cb, clen = len(words), 256, 1000
    letters = torch.tensor([i for w in words for i in w], dtype=torch.int64, device="cuda:0")
    degrees = torch.full((n_words,), 3, dtype=torch.int64, device="cuda:0")
    cpath = torch.rand((cb, clen, d), **f64)
    cout = torch.empty((cb, 3 * n_words), **f64)
    cg = torch.rand((cb, 3 * n_words), **f64)
    cgrad = torch.empty_like(cpath)

    sig_bytes = batch * n * 8
    cases = [
        ("sig_combine", lambda: loader.CUSIG_SIG_COMBINE["float64"](p(a), p(b), p(o1), batch, d, deg, False), 3 * sig_bytes),
        ("sig_combine_backprop", lambda: loader.CUSIG_SIG_COMBINE_BACKPROP["float64"](p(g), p(o1), p(o2), p(a), p(b), batch, d, deg, False), 5 * sig_bytes),
        ("linear_sig", lambda: loader.CUSIG_LINEAR_SIG["float64"](p(z), p(o1), batch, d, deg, False), sig_bytes),
        ("sig_join", lambda: loader.CUSIG_SIG_JOIN["float64"](p(a), p(z), p(o1), batch, d, deg, False, False), 2 * sig_bytes),
        ("sig_join_backprop", lambda: loader.CUSIG_SIG_JOIN_BACKPROP["float64"](p(g), p(o1), p(oz), p(a), p(z), batch, d, deg, False, False), 3 * sig_bytes),
        ("sig_to_log_sig", lambda: loader.CUSIG_SIG_TO_LOG_SIG["float64"](p(a), p(o1), batch, d, deg, 0, False), 2 * sig_bytes),
        ("sig_to_log_sig_backprop", lambda: loader.CUSIG_SIG_TO_LOG_SIG_BACKPROP["float64"](p(a), p(o1), p(g), batch, d, deg, 0, False), 3 * sig_bytes),
        ("sig_coef", lambda: loader.CUSIG_SIG_COEF["float64"](p(cpath), p(cout), pu(letters), n_words, pu(degrees), cb, d, clen, True), (cpath.numel() + cout.numel()) * 8),
        ("sig_coef_backprop", lambda: loader.CUSIG_SIG_COEF_BACKPROP["float64"](p(cpath), p(cgrad), p(cout), p(cg), pu(letters), n_words, pu(degrees), cb, d, clen), (2 * cpath.numel() + 2 * cout.numel()) * 8),
        ("transform_path", lambda: loader.CUSIG_TRANSFORM_PATH["float64"](p(path), p(tpath), pb, pdim, plen, True, True, 1.0), (path.numel() + tpath.numel()) * 8),
        ("transform_path_backprop", lambda: loader.CUSIG_TRANSFORM_PATH_BACKPROP["float64"](p(tpath), p(gpath), pb, pdim, plen, True, True, 1.0), (path.numel() + tpath.numel()) * 8),
    ]
    out = {}
    for name, fn, nbytes in cases:
        for _ in range(args.warmup):
            rc = fn()
            if rc:
                raise RuntimeError("%s failed: %d %s" % (name, rc, loader.last_error_message()))
        times = []
        for _ in range(args.steps):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        ms = statistics.median(times) * 1e3
        out[name] = {"call_ms": ms, "algorithmic_bytes": nbytes, "GB_per_s": nbytes / (ms * 1e-3) / 1e9,
                     "hbm_frac": nbytes / (ms * 1e-3) / 8e12}
    print(json.dumps({"metric": "operator kernels, achieved HBM GB/s (algorithmic bytes / synchronous call time)",
                      "unit": "GB/s", "peak": 8000.0, "dtype": "f64", "data": "synthetic", "steps": args.steps,
                      "warmup": args.warmup,
                      "config": {"workload": "signatures: batch %d, dim %d, degree %d (%d coefficients); paths: (%d, %d, %d) "
                                             "with lead-lag + time; sig_coef: %d words of 3 letters, paths (%d, %d, %d) "
                                             "(a sweep: compute-bound, its GB/s is not a bandwidth figure)"
                                             % (batch, d, deg, n, pb, plen, pdim, n_words, cb, clen, d)},
                      "ops": out}))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (batch sharding needs no communication and is left to the "
              "caller); re-run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    from pysiglib_amd import _loader as loader
    from pysiglib_amd import workloads as cfgmod

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    if args.copy_calib:
        n = 256 * 1024 * 1024 // 8
        src = torch.arange(n, dtype=torch.float64, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)          # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        print(json.dumps({"copy_calib_bytes_read": n * 8, "copy_calib_bytes_written": n * 8, "copies": 3}))
        return

    if args.ops:
        bench_ops(args, torch, loader)
        return

    r1 = Runner(1, torch, np, loader, cfgmod)
    r5 = Runner(5, torch, np, loader, cfgmod)
    r5.forward()            # the backward consumes the forward's signature
    torch.cuda.synchronize()
    peak = PEAK_TFLOPS["float64"]
    configs = {}

    if not args.headline_only:      # all five workloads by default (a few seconds more); the headline comes last
        for k in (2, 3, 4):
            r = Runner(k, torch, np, loader, cfgmod)
            n = 3 if k == 3 else max(5, min(args.steps, 50))
            wall, kms, name = time_calls(r.forward, torch, loader, 1, n)
            tf = r.flops_fwd / (kms * 1e-3) / 1e12
            configs["C%d" % k] = {"signatures_per_s": r.c["batch"] / wall, "call_ms": wall * 1e3, "kernel": name,
                                  "kernel_ms": kms, "tflops": tf, "roofline_frac": tf / PEAK_TFLOPS[r.dtype],
                                  # the whole call (sweep plus, when the paths were cut in time, the Chen folds)
                                  "call_roofline_frac": r.flops_fwd / wall / 1e12 / PEAK_TFLOPS[r.dtype],
                                  "time_segments": int(loader.CUSIG.cusig_amd_last_segments())}
            if name.endswith("_ll"):
                configs["C%d" % k]["note"] = ("flops are those of the dense sweep over all augmented channels (the reference's "
                                              "arithmetic); this kernel leaves out the multiply-adds by the channels a lead-lag "
                                              "step cannot move, so tflops / roofline_frac are effective rates, not pipe utilisation")
            del r
            torch.cuda.empty_cache()
        # degree 2 on paths of many channels: closed form on the matrix cores (not one of the five benchmark workloads)
        db, dl, dd = 2048, 256, 64
        xp = (torch.randn((db, dl, dd), dtype=torch.float32, device="cuda:0").cumsum(1) * 0.05).contiguous()
        sg = torch.empty((db, dd + dd * dd), dtype=torch.float32, device="cuda:0")
        gg = torch.randn_like(sg)
        gx = torch.empty_like(xp)
        fp = ctypes.POINTER(ctypes.c_float)

        def d2_fwd():
            loader.CUSIG_SIGNATURE["float32"](ctypes.cast(xp.data_ptr(), fp), ctypes.cast(sg.data_ptr(), fp), db, dd, dl, 2,
                                              False, False, 1.0, True, False, None, 0, 0, 0)

        def d2_bwd():
            loader.CUSIG_SIG_BACKPROP["float32"](ctypes.cast(xp.data_ptr(), fp), ctypes.cast(gx.data_ptr(), fp),
                                                 ctypes.cast(gg.data_ptr(), fp), ctypes.cast(sg.data_ptr(), fp), db, dd, dl,
                                                 2, False, False, 1.0, False, None, 0, 0, 0)

        mm_flops = 2.0 * db * (dl - 1) * dd * dd        # one (d x L)(L x d) resp. (L x d)(d x d) product per path
        for tag, fn in (("D2 fwd f32 (2048,256,64) deg 2", d2_fwd), ("D2 bwd f32 (2048,256,64) deg 2", d2_bwd)):
            wall, kms, name = time_calls(fn, torch, loader, 2, max(5, min(args.steps, 50)))
            configs[tag] = {"signatures_per_s": db / wall, "call_ms": wall * 1e3, "kernel": name, "kernel_ms": kms,
                            "tflops": mm_flops / (kms * 1e-3) / 1e12, "bound": "mfma",
                            "roofline_frac": mm_flops / (kms * 1e-3) / 1e12 / PEAK_TFLOPS["float32"]}
        del xp, sg, gg, gx
        torch.cuda.empty_cache()
        # further f32 legs, none of them one of the five benchmark workloads: degree 3 on paths of many channels (the
        # backward as two library matrix products around a scan), a shape the instance table reaches at degree 6, and
        # one beyond the table (run-time-dimension kernels); flops are the sweep's operation count, as for the workloads
        for prefix, tb, tl, td, tdeg in (("D3", 512, 256, 80, 3), ("T6", 64, 200, 10, 6), ("R4", 16, 200, 64, 4)):
            xp = (torch.randn((tb, tl, td), dtype=torch.float32, device="cuda:0").cumsum(1) * (0.5 / tl ** 0.5)).contiguous()
            sg = torch.empty((tb, int(loader.CUSIG.cusig_amd_sig_length(td, tdeg)) - 1), dtype=torch.float32, device="cuda:0")
            gg = torch.randn_like(sg)
            gx = torch.empty_like(xp)

            def leg_fwd():
                loader.CUSIG_SIGNATURE["float32"](ctypes.cast(xp.data_ptr(), fp), ctypes.cast(sg.data_ptr(), fp), tb, td, tl,
                                                  tdeg, False, False, 1.0, True, False, None, 0, 0, 0)

            def leg_bwd():
                loader.CUSIG_SIG_BACKPROP["float32"](ctypes.cast(xp.data_ptr(), fp), ctypes.cast(gx.data_ptr(), fp),
                                                     ctypes.cast(gg.data_ptr(), fp), ctypes.cast(sg.data_ptr(), fp), tb, td, tl,
                                                     tdeg, False, False, 1.0, False, None, 0, 0, 0)

            shape = "f32 (%d,%d,%d) deg %d" % (tb, tl, td, tdeg)
            for tag, fn, fl in (("%s fwd %s" % (prefix, shape), leg_fwd, cfgmod.flops_fwd(td, tdeg)),
                                ("%s bwd %s" % (prefix, shape), leg_bwd, cfgmod.flops_bwd(td, tdeg))):
                wall, kms, name = time_calls(fn, torch, loader, 2, 5)
                tf = tb * (tl - 1) * fl / (kms * 1e-3) / 1e12
                configs[tag] = {"signatures_per_s": tb / wall, "call_ms": wall * 1e3, "kernel": name, "kernel_ms": kms,
                                "tflops": tf, "roofline_frac": tf / PEAK_TFLOPS["float32"]}
                if "degree3" in name:
                    configs[tag]["note"] = ("runs as matrix products on the matrix cores around a scan: tflops is the sweep's "
                                            "operation count over the time (a sweep-equivalent rate), and roofline_frac sets "
                                            "it against the vector FP32 peak the sweep would be bound by; neither is a "
                                            "utilisation of the matrix pipe")
            del xp, sg, gg, gx
            torch.cuda.empty_cache()

    def step():
        r1.forward()
        r5.backward()

    # the same steps with the library in stream-ordered mode (calls only enqueue, the host syncs once at the end).  The
    # legs before it end with long kernels that leave the clocks low: it gets a longer warm-up of its own, and in turn
    # leaves the device in the state the headline is measured in.
    loader.CUSIG.cusig_amd_set_stream_ordered.argtypes = (ctypes.c_int,)
    loader.CUSIG.cusig_amd_set_stream_ordered.restype = None
    loader.CUSIG.cusig_amd_set_stream_ordered(1)
    try:
        for _ in range(max(args.warmup, 50)):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ordered_ms = (time.perf_counter() - t0) / args.steps * 1e3
    finally:
        loader.CUSIG.cusig_amd_set_stream_ordered(0)
        torch.cuda.synchronize()

    # per-kernel figures of the same two calls (HIP events inside the library, on the launch stream)
    wall_f, kms_f, name_f = time_calls(r1.forward, torch, loader, 3, max(5, args.steps))
    wall_b, kms_b, name_b = time_calls(r5.backward, torch, loader, 3, max(5, args.steps))
    tf_f = r1.flops_fwd / (kms_f * 1e-3) / 1e12
    tf_b = r5.flops_bwd / (kms_b * 1e-3) / 1e12
    # the headline comes after every other leg on the sweep kernels, so that it is timed on a device in steady state
    ms_per_step, ms_mean = time_steps(step, torch, args.warmup, args.steps)
    value = r1.c["batch"] / (ms_per_step * 1e-3)


    # the Python wrappers on the same device tensors: argument checks, output allocation, the overflow report
    import pysiglib_amd
    x1, g5, s5 = r1.path, r5.gsig, r5.sig

    def wrapped(fn):
        for _ in range(5):
            fn()
        each = []
        for _ in range(max(10, min(args.steps, 100))):
            t0 = time.perf_counter()
            fn()
            each.append(time.perf_counter() - t0)
        return statistics.median(each) * 1e3

    wrap_f = wrapped(lambda: pysiglib_amd.sig(x1, r1.c["degree"]))
    wrap_b = wrapped(lambda: pysiglib_amd.sig_backprop(x1, s5, g5, r5.c["degree"]))
    peaks = measured_peaks(loader)      # last: its sustained full-rate kernels leave the clocks lower than they found them
    dominant = {"kernel": name_b, "ms": kms_b, "tflops": tf_b} if kms_b >= kms_f else {"kernel": name_f, "ms": kms_f, "tflops": tf_f}
    headline = {
        "C1": {"signatures_per_s": r1.c["batch"] / wall_f, "call_ms": wall_f * 1e3, "python_wrapper_call_ms": wrap_f,
               "kernel": name_f, "kernel_ms": kms_f, "tflops": tf_f, "roofline_frac": tf_f / peak},
        "C5": {"signatures_per_s": r5.c["batch"] / wall_b, "call_ms": wall_b * 1e3, "python_wrapper_call_ms": wrap_b,
               "kernel": name_b, "kernel_ms": kms_b, "tflops": tf_b, "roofline_frac": tf_b / peak},
    }
    headline.update(configs)
    configs = headline

    line = {
        "metric": "signatures/sec, (32,1000,10) deg 5 fwd+bwd, fp64, 1 GPU",
        "value": value,
        "unit": "signatures/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_mean": ms_mean,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": "sig forward + sig_backprop, batch 32, length 1000, dim 10, degree 5, float64, "
                               "points iid N(0,1) seed 1001; upstream grad iid N(0,1)"},
        "roofline": {
            "bound": "vector_fp64", "pipe": "vector FP64 FMA (per-path rank-1 updates and GEMVs: no MFMA tile applies)",
            "kernel": dominant["kernel"], "achieved": dominant["tflops"], "peak": peak, "unit": "TFLOP/s",
            "frac": dominant["tflops"] / peak, "kernel_ms": dominant["ms"],
            "traffic": traffic_bytes(dominant["kernel"]),
            # measured ceilings (independent FMAs only): the chip's best, and what one wave per SIMD, the regime of
            # this workload's 1024 waves, can issue
            "measured_peak": dict(peaks, unit="TFLOP/s"),
            "frac_of_measured": (dominant["tflops"] / peaks["f64"]["8_waves_per_simd"]) if peaks["f64"]["8_waves_per_simd"] else None,
            "frac_of_measured_one_wave_per_simd": (dominant["tflops"] / peaks["f64"]["1_waves_per_simd"])
            if peaks["f64"]["1_waves_per_simd"] else None,
            "fwd_bwd_combined_frac": (r1.flops_fwd + r5.flops_bwd) / ((kms_f + kms_b) * 1e-3) / 1e12 / peak,
            # the whole synchronous step as timed above (launches and host waits included)
            "step_frac": (r1.flops_fwd + r5.flops_bwd) / (ms_per_step * 1e-3) / 1e12 / peak,
        },
        "configs": configs,
        "stream_ordered": {"value": r1.c["batch"] / (ordered_ms * 1e-3), "ms_per_step": ordered_ms,
                           "note": "same steps with cusig_amd_set_stream_ordered(1): calls enqueue on the null stream, "
                                   "one host synchronisation after the last step; `value` above is the reference's "
                                   "synchronous contract"},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(np, cfgmod)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
