"""Benchmark of the matmul training core on one MI355X.

One step = forward + weight gradient + input gradient of the Linear 1024 -> 1024 layer in fp16 (fp32
accumulation) over a batch of 512 independent samples (BASELINE.json configs[1], batched mode), called through
the C ABI of libptl_hip.so with every tensor already resident in HBM.

The LAST line of stdout is one compact JSON object (a few KB at most) that carries
  * "roofline": the dominant kernel (the MFMA GEMM) priced against the dense fp16 MFMA peak, from HIP events
    recorded on the library's stream around the timed region;
  * "cpu_baseline": the CPU oracle (a port of the reference's C loops, OpenMP over the host cores) timed on a
    bounded sample of the same workload;
  * "targets": a handful of figures of the other BASELINE shapes (wide convolutions, a large plain product,
    depthwise / pointwise at batch 64, the ResNet-20 step).
Everything else -- the per-step timings of every other shape (batch-1 latency and batched mode) with their own
roofline fractions, and the CPU port on every configuration -- is printed BEFORE it, one JSON object per line
(`{"detail": {...}}`, `{"cpu_baseline_detail": {...}}`), and with --detail-file also written to a file.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK = {"fp16": 2500.0, "fp32": 157.3}  # dense MFMA TFLOP/s
HBM_GBS = 8000.0
METRIC = "Conv2D/Linear FW+WG+IG TFLOP/s & % MFMA peak (fp32/fp16); samples/s"


TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_plain_f16_linear1024_N512.md")
TRAFFIC_SOURCES = ["ptl_gemm_plain.inc", "ptl_gemm_async.inc", "ptl_gemm_async_sel.hip", "ptl_gemm_plain_f16.hip"]


def kernel_sources_digest():
    """sha256 over the sources of the headline kernels and their selection."""
    import hashlib
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, "pulp-trainlib_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def recorded_traffic(ns):
    """(bytes per launch, note): the HBM traffic the counter runs measured for the headline launches, as
    recorded in the profile summary (a line `roofline.traffic: bytes_per_launch=... batch=... sources=...`)."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            lines = [l for l in f if l.startswith("roofline.traffic:")]
        fields = dict(kv.split("=") for kv in lines[-1].split()[1:])
        if int(fields["batch"]) != ns:
            return None, "counters were collected at batch %s" % fields["batch"]
        if fields["sources"] != kernel_sources_digest():
            return None, "kernel sources changed since the counter runs (recorded %s)" % fields["sources"]
        return float(fields["bytes_per_launch"]), None
    except (OSError, IndexError, KeyError, ValueError) as e:
        return None, "no usable traffic record (%s)" % type(e).__name__


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-detail", action="store_true", help="skip the per-shape detail table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--detail-file", default=None,
                    help="also write the headline, the CPU table and the detail table to this file as one JSON document")
    ap.add_argument("--helpers-only", action="store_true",
                    help="detail table: only the index / streaming helpers (for a counter run of those kernels alone)")
    ap.add_argument("--resnet-only", action="store_true",
                    help="detail table: only the ResNet-20-shaped step (for a kernel trace of that step alone)")
    ap.add_argument("--batch", type=int, default=512, help="samples per step of the headline workload")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run a 64 MiB device copy five times (a kernel of known traffic, to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported "
              "(the path shards by sample; no multi-GPU figure is produced)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import __graft_entry__ as ge
    import helpers as hp

    pkg = ge.load_package()
    lib = pkg.load()  # raises if libptl_hip.so is not built
    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs a GPU")
    if lib.ptl_init(0) != 0:
        raise RuntimeError(lib.ptl_last_error().decode())
    dev = torch.device("cuda:0")

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.ptl_last_error().decode())

    def to_dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def timed(fn, iters, warm=5):
        """Average milliseconds per call of fn, by HIP events on the library stream."""
        for _ in range(warm):
            fn()
        check(lib.ptl_sync())
        check(lib.ptl_timer_begin())
        for _ in range(iters):
            fn()
        ms = lib.ptl_timer_end_ms()
        if ms < 0:
            raise RuntimeError(lib.ptl_last_error().decode())
        return ms / iters

    if args.copy_calib:
        nbytes = 64 << 20
        src = torch.ones(nbytes // 4, dtype=torch.float32, device=dev)
        dst = torch.zeros_like(src)
        for _ in range(5):
            check(lib.ptl_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes))
        check(lib.ptl_sync())

    # ------------------------------------------------------------------ headline workload
    n_in = n_out = 1024
    ns = args.batch
    dt, nd = "fp16", np.float16
    seed = 0xC0DE0002
    x = hp.normal(seed, (ns, n_in), 1.0 / 32.0, nd)
    w = hp.normal(seed + 1, (n_out, n_in), 1.0 / 32.0, nd)
    dy = hp.uniform(seed + 2, (ns, n_out), dtype=nd)
    gx, gw, gdy = to_dev(x), to_dev(w), to_dev(dy)
    gy = torch.zeros(ns, n_out, dtype=torch.float16, device=dev)
    gdx = torch.zeros(ns, n_in, dtype=torch.float16, device=dev)
    gdw = torch.zeros(n_out, n_in, dtype=torch.float16, device=dev)
    la, keep = hp.linear_args(pkg, gx, gdx, gw, gdw, gy, gdy, n_in, n_out)
    import ctypes
    la_ref = ctypes.byref(la)
    # The reference drives a layer with a forward call and ONE backward call that produces both gradients
    # (pulp_linear_fp16_fw_cl, pulp_linear_fp16_bw_cl); the batched twins are used the same way.
    fw, bw = lib.ptl_linear_fp16_fw_batched, lib.ptl_linear_fp16_bw_batched

    def step():
        check(fw(la_ref, ns))
        check(bw(la_ref, ns))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    check(lib.ptl_timer_begin())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    ev_ms = lib.ptl_timer_end_ms()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    flops_step = 3 * 2.0 * ns * n_in * n_out
    tflops = flops_step / (ms_per_step * 1e-3) / 1e12
    # Two launches per step: the forward product, and weight + input gradient sharing one launch.  The
    # roofline prices the three products of a step against the event time of the step.
    launches = 2 * args.steps
    launch_ms = ev_ms / launches
    achieved = flops_step / (2 * launch_ms * 1e-3) / 1e12

    traffic, traffic_note = recorded_traffic(ns)

    cpu_detail, detail = [], []
    result = {
        "metric": METRIC,
        "value": round(tflops, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "samples_per_s": round(ns / (ms_per_step * 1e-3), 1),
        "config": {"workload": "linear_1024x1024_fp16_FW+WG+IG_batched_N%d" % ns, "in": n_in, "out": n_out,
                   "batch": ns, "accumulate": "f32", "layout": "W[out][in], X[batch][in]"},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK["fp16"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK["fp16"], 5),
                     # HBM bytes per launch (mean of the two launches of a step), from the FETCH_SIZE and
                     # WRITE_SIZE counter runs recorded in the profile summary of this workload; null when the
                     # batch differs or the kernel sources have changed since those runs
                     "traffic": traffic,
                     "kernel": "ptl::gemm_plain_kernel<_Float16, 64x64 tile, 1024 threads> / gemm_plain_pair_mixed_kernel<_Float16> (128x64 and 64x64 tiles)",
                     "flops_per_launch": flops_step / 2, "launches_per_step": 2,
                     "avg_launch_us": round(launch_ms * 1e3, 3)},
    }

    if traffic_note:
        result["roofline"]["traffic_note"] = traffic_note
    # `value` is wall-clock over the timed steps (launch overhead of the calling thread included);
    # `roofline.achieved` prices the same steps against HIP event time on the library's stream.
    result["roofline"]["event_ms_per_step"] = round(ev_ms / args.steps, 6)

    # The same step handed over as host buffers (the library stages them: allocate, copy in, run, copy out).
    # Reported beside the headline, never as the headline.
    hy, hdx, hdw = np.zeros((ns, n_out), nd), np.zeros((ns, n_in), nd), np.zeros((n_out, n_in), nd)
    ha, hkeep = hp.linear_args(pkg, x, hdx, w, hdw, hy, dy, n_in, n_out)
    ha_ref = ctypes.byref(ha)
    for _ in range(2):
        check(fw(ha_ref, ns)); check(bw(ha_ref, ns))
    t0 = time.perf_counter()
    for _ in range(5):
        check(fw(ha_ref, ns)); check(bw(ha_ref, ns))
    host_ms = (time.perf_counter() - t0) * 1e3 / 5
    result["host_staged"] = {"ms_per_step": round(host_ms, 4), "TFLOP/s": round(flops_step / (host_ms * 1e-3) / 1e12, 3),
                             "note": "same step with host pointers: per call hipMalloc + H2D + kernel + D2H + sync"}

    # ------------------------------------------------------------------------ CPU baseline
    if not args.no_cpu:
        orc = ge.load_oracle()
        olib = orc.load()
        # the reference's own core count (NUM_CORES = 8, tests/test_conv2d_fp32/Makefile:16), clamped to the host
        olib.orc_set_num_threads(min(8, os.cpu_count() or 8))
        cores = int(olib.orc_num_threads())

        def cpu_step(m):
            y = np.zeros((m, n_out), nd)
            dx = np.zeros((m, n_in), nd)
            dw_ = np.zeros((n_out, n_in), nd)
            a, k2 = hp.linear_args(pkg, x[:m].copy(), dx, w, dw_, y, dy[:m].copy(), n_in, n_out)
            t = time.perf_counter()
            for s in ("fw", "wg", "ig"):
                orc.call("orc_linear_" + s, dt, a, m)
            return time.perf_counter() - t

        cpu_step(2)
        t_probe = cpu_step(4) / 4
        m = int(max(4, min(ns, 12.0 / max(t_probe, 1e-6))))
        reps = int(max(1, min(50, round(10.0 / max(t_probe * m, 1e-6)))))  # about 10 s of CPU work
        t_cpu = sum(cpu_step(m) for _ in range(reps))
        cpu_tflops = reps * 3 * 2.0 * m * n_in * n_out / t_cpu / 1e12
        result["cpu_baseline"] = {"value": round(cpu_tflops, 6), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                                  "sample": "%d of the %d samples, FW+WG+IG %d times, fp16 with fp16 accumulation "
                                            "(the reference's arithmetic), %.2f s" % (m, ns, reps, t_cpu)}
        cpu_detail = cpu_rows(pkg, orc, hp, cores)

    # ------------------------------------------------------------------------------ detail
    if args.helpers_only:
        detail = helper_rows(pkg, lib, hp, timed, torch, dev)
    elif args.resnet_only:
        detail = resnet_rows(pkg, lib, timed, torch, dev)
    elif not args.no_detail:
        detail = detail_table(pkg, lib, hp, to_dev, timed, check, torch, dev)

    lines = compose_output(result, cpu_detail, detail)
    if args.detail_file:
        with open(args.detail_file, "w") as f:
            json.dump({"headline": result, "cpu_baseline_detail": cpu_detail, "detail": detail}, f, indent=1)
    for line in lines:
        print(line)
    sys.stdout.flush()


# (key of the "targets" block, workload names in the detail table -- matched as prefixes --, field reported)
TARGET_ROWS = (
    ("conv512_14x14_N256_FW_WG_IG_frac_of_mfma_peak",
     ["conv2d 512->512 14x14 k3 p1 %s N=256" % s for s in ("FW", "WG", "IG")], "frac_of_bound"),
    ("conv256_28x28_N256_FW_WG_IG_frac_of_mfma_peak",
     ["conv2d 256->256 28x28 k3 p1 %s N=256" % s for s in ("FW", "WG", "IG")], "frac_of_bound"),
    ("conv128_28x28_N512_FW_WG_IG_frac_of_mfma_peak",
     ["conv2d 128->128 28x28 k3 p1 %s N=512" % s for s in ("FW", "WG", "IG")], "frac_of_bound"),
    ("conv256_28x28_N256_FW_input_copy_handed_on_frac_of_mfma_peak",
     ["conv2d 256->256 28x28 k3 p1 FW, input copy left by the layer before N=256"], "frac_of_bound"),
    ("mm_4096x4096x4096_fp16_TFLOP/s", ["mm 4096x4096x4096 (B transposed)"], "TFLOP/s"),
    ("depthwise_64x56x56_N64_FW_WG_IG_GB/s", ["depthwise 3x3 64x56x56 %s N=64" % s for s in ("FW", "WG", "IG")], "GB/s"),
    ("pointwise_64to128_56x56_N64_FW_WG_IG_GB/s", ["pointwise 64->128 56x56 %s N=64" % s for s in ("FW", "WG", "IG")], "GB/s"),
    ("mhsa_L197_E192_N32_FW_BW_us", ["mhsa L197 E192 3x64 %s N=32" % s for s in ("FW", "BW")], "us"),
    ("resnet20_fp16_N128_step_samples/s",
     ["resnet20 step with batch norm, element-wise layers fused into it, its sums formed by the convolutions in both passes, "
      "applied inside the forward convolutions, pooling + classifier + loss in one call"],
     "samples/s"),
    ("mm_4096_fp16_random_then_zero_operands_TFLOP/s",
     ["power: mm 4096x4096x4096 (B transposed), random", "power: mm 4096x4096x4096 (B transposed), zero"], "TFLOP/s"),
)
MAX_LAST_LINE = 4096


def compose_output(result, cpu_detail, detail):
    """The lines bench.py prints, in order: one JSON object per row of the CPU table and of the detail table, then
    the headline object LAST, kept under MAX_LAST_LINE bytes so that a reader that only sees the tail of stdout
    still gets it whole.  Strict JSON throughout (a NaN or an infinity raises)."""
    lines = []
    for row in cpu_detail or ():
        lines.append(json.dumps({"cpu_baseline_detail": row}, allow_nan=False))
    for row in detail or ():
        lines.append(json.dumps({"detail": row}, allow_nan=False))
    head = dict(result)
    targets = {}
    for key, names, field in TARGET_ROWS:
        vals = []
        for name in names:
            hit = [row for row in detail or () if row["workload"].startswith(name) and field in row]
            vals.append(hit[0][field] if hit else None)
        if any(v is not None for v in vals):
            targets[key] = vals if len(vals) > 1 else vals[0]
    if targets:
        head["targets"] = targets
    last = json.dumps(head, allow_nan=False)
    if len(last) >= MAX_LAST_LINE:
        raise RuntimeError("headline line is %d bytes, limit %d" % (len(last), MAX_LAST_LINE))
    lines.append(last)
    return lines


class PowerSampler:
    """Board power from the amdgpu hwmon node (microwatts in power1_input / power1_average), read every 10 ms on a
    thread while a workload runs.  None when the node is not there."""

    def __init__(self):
        import glob
        self.path = self.cap = None
        for h in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
            for n in ("power1_input", "power1_average"):
                if self.path is None and os.path.exists(os.path.join(h, n)):
                    self.path = os.path.join(h, n)
                    try:
                        self.cap = int(open(os.path.join(h, "power1_cap")).read()) / 1e6
                    except (OSError, ValueError):
                        self.cap = None

    def run(self, fn, sync, secs=1.0):
        """Calls fn back to back for `secs` seconds; returns (microseconds per call, mean watts over the last two
        thirds of the samples or None)."""
        import threading
        for _ in range(3):
            fn()
        sync()
        samples, stop = [], [False]

        def loop():
            while not stop[0]:
                try:
                    samples.append(int(open(self.path).read()) / 1e6)
                except (OSError, ValueError):
                    pass
                time.sleep(0.01)
        th = threading.Thread(target=loop) if self.path else None
        if th:
            th.start()
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < secs:
            for _ in range(20):
                fn()
            sync()
            n += 20
        dt = time.perf_counter() - t0
        stop[0] = True
        if th:
            th.join()
        tail = samples[len(samples) // 3:]
        return dt / n * 1e6, (sum(tail) / len(tail) if tail else None)


def power_rows(pkg, lib, hp, check, torch, dev):
    """The same launches on random and on all-zero operands, with the board power read beside them.  On random
    operands the matrix kernels run against the board's power limit (the clock drops until the power fits), on zeros
    they do not: the difference is what the limit, not the kernel's pipeline, takes."""
    import ctypes
    rows = []
    ps = PowerSampler()
    sync = torch.cuda.synchronize
    N = 4096
    ns, Ci, Co, H = 256, 512, 512, 14
    # what the matrix cores sustain on a loop of nothing but MFMAs (no loads, no LDS): the ceiling on that data
    for shape in (32, 16):
        for kind in ("random", "zero"):
            for waves in (1, 2):
                tf = ctypes.c_float(0)

                def probe():
                    check(lib.ptl_probe_mfma_fp16(shape, 1 if kind == "random" else 0, waves, 4000, ctypes.byref(tf)))
                us, w = ps.run(probe, sync, 0.4)
                rows.append({"workload": "power: loop of v_mfma_f32_%s_f16 alone, %s operands, %d wave%s per SIMD"
                                         % ("32x32x16" if shape == 32 else "16x16x32", kind, waves, "s" if waves > 1 else ""),
                             "dtype": "fp16", "us": round(us, 2), "TFLOP/s": round(tf.value, 1),
                             "W": None if w is None else round(w), "cap_W": ps.cap})
    for kind in ("random", "zero"):
        def mk(*shape):
            if kind == "zero":
                return torch.zeros(*shape, device=dev, dtype=torch.float16)
            return (torch.rand(*shape, device=dev) - 0.5).to(torch.float16)
        A, Bm, Cm = mk(N, N), mk(N, N), torch.zeros(N, N, device=dev, dtype=torch.float16)
        margs = [ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(Bm.data_ptr()), ctypes.c_void_p(Cm.data_ptr()), N, N, N, 1]
        us, w = ps.run(lambda: check(lib.ptl_mm_fp16(*margs)), sync)
        rows.append({"workload": "power: mm 4096x4096x4096 (B transposed), %s operands" % kind, "dtype": "fp16",
                     "us": round(us, 2), "TFLOP/s": round(2.0 * N ** 3 / us / 1e6, 1),
                     "W": None if w is None else round(w), "cap_W": ps.cap})
        del A, Bm, Cm
        x, wt = mk(ns, Ci, H, H), mk(Co, Ci, 3, 3)
        y = torch.zeros(ns, Co, H, H, device=dev, dtype=torch.float16)
        a, keep = hp.conv2d_args(pkg, x, None, wt, None, y, None, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1))
        ref = ctypes.byref(a)
        us, w = ps.run(lambda: check(lib.ptl_conv2d_fp16_fw_batched(ref, ns)), sync)
        rows.append({"workload": "power: conv2d 512->512 14x14 k3 p1 FW N=256, %s operands" % kind, "dtype": "fp16",
                     "us": round(us, 2), "TFLOP/s": round(2.0 * ns * Co * Ci * 9 * H * H / us / 1e6, 1),
                     "W": None if w is None else round(w), "cap_W": ps.cap})
        del x, wt, y
    # and on operands shaped like a trained network's: the input a rectified Gaussian (half of it zeros), small
    # Gaussian filters - between the two above in the power they draw
    x = torch.relu(torch.randn(ns, Ci, H, H, device=dev)).to(torch.float16)
    wt = (torch.randn(Co, Ci, 3, 3, device=dev) * 0.03).to(torch.float16)
    y = torch.zeros(ns, Co, H, H, device=dev, dtype=torch.float16)
    a, keep = hp.conv2d_args(pkg, x, None, wt, None, y, None, Ci, H, H, Co, 3, 3, H, H, (1, 1, 1, 1))
    ref = ctypes.byref(a)
    us, w = ps.run(lambda: check(lib.ptl_conv2d_fp16_fw_batched(ref, ns)), sync)
    rows.append({"workload": "power: conv2d 512->512 14x14 k3 p1 FW N=256, rectified-Gaussian input, Gaussian filters",
                 "dtype": "fp16", "us": round(us, 2), "TFLOP/s": round(2.0 * ns * Co * Ci * 9 * H * H / us / 1e6, 1),
                 "W": None if w is None else round(w), "cap_W": ps.cap})
    del x, wt, y
    return rows


def cpu_rows(pkg, orc, hp, cores):
    """The CPU oracle (a port of the reference's loops, OpenMP over `cores` threads) on the other BASELINE
    configurations, one sample each where the batched mode is a loop over samples: microseconds and TFLOP/s per
    step, median of a bounded number of repetitions (about a second per row)."""
    import ctypes
    rows = []

    def median_time(fn, budget=0.6, max_reps=21):
        fn()
        times = []
        t_all = time.perf_counter()
        while len(times) < max_reps and (len(times) < 3 or time.perf_counter() - t_all < budget):
            t = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t)
        times.sort()
        return times[len(times) // 2], len(times)

    def add(name, dt, flops, fn):
        t, reps = median_time(fn)
        rows.append({"workload": name, "dtype": dt, "us": round(t * 1e6, 1), "TFLOP/s": round(flops / t / 1e12, 6),
                     "threads": cores, "kind": "port", "sample": "one call, median of %d" % reps})

    for dt in ("fp32", "fp16"):  # config 1
        nd = hp.np_dtype(dt)
        Ci, Co, H, K = 16, 32, 32, 3
        x, w, dy = hp.uniform(1, (Ci, H, H), dtype=nd), hp.uniform(2, (Co, Ci, K, K), dtype=nd), hp.uniform(3, (Co, H, H), dtype=nd)
        y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
        for s in ("fw", "wg", "ig"):
            add("conv2d 16->32 32x32 k3 p1 %s N=1" % s.upper(), dt, 2.0 * Co * Ci * K * K * H * H,
                lambda s=s: orc.call("orc_conv2d_" + s, dt, a, 1))
    for dt in ("fp32", "fp16"):  # config 2, one sample (batched mode on the CPU = a loop over samples)
        nd = hp.np_dtype(dt)
        n = 1024
        x, w, dy = hp.normal(4, (n,), 1 / 32.0, nd), hp.normal(5, (n, n), 1 / 32.0, nd), hp.uniform(6, (n,), dtype=nd)
        y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
        a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n, n)
        for s in ("fw", "wg", "ig"):
            add("linear 1024x1024 %s N=1" % s.upper(), dt, 2.0 * n * n, lambda s=s: orc.call("orc_linear_" + s, dt, a, 1))
    dt, nd = "fp16", np.float16  # config 3
    C, Hp, Ho, K = 64, 58, 56, 3
    x, w, dy = hp.uniform(7, (C, Hp, Hp), dtype=nd), hp.uniform(8, (C, K, K), dtype=nd), hp.uniform(9, (C, Ho, Ho), dtype=nd)
    y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
    a3, keep3 = hp.dw_args(pkg, dt, x, dx, w, dw, y, dy, C, Hp, Hp, K, K, Ho, Ho)
    for s in ("fw", "wg", "ig"):
        add("depthwise 3x3 64x56x56 %s N=1" % s.upper(), dt, 2.0 * C * K * K * Ho * Ho,
            lambda s=s: orc.call("orc_conv_dw_" + s, dt, a3, 1))
    Ci, Co, H = 64, 128, 56
    x, w, dy = hp.uniform(10, (Ci, H * H), dtype=nd), hp.uniform(11, (Co, Ci), dtype=nd), hp.uniform(12, (Co, H * H), dtype=nd)
    y, dx, dw = np.zeros_like(dy), np.zeros_like(x), np.zeros_like(w)
    a4, keep4 = hp.pw_args(pkg, x, dx, w, dw, y, dy, Ci, Co, H, H)
    for s in ("fw", "wg", "ig"):
        add("pointwise 64->128 56x56 %s N=1" % s.upper(), dt, 2.0 * Co * Ci * H * H,
            lambda s=s: orc.call("orc_conv_pw_" + s, dt, a4, 1))
    # config 4: attention step, one sequence
    L, E, F, heads = 197, 192, 192, 3
    sh = hp.mhsa_shapes(1, L, E, F, heads)
    d, dyh = hp.mhsa_inputs(0xC0DE0004, 1, L, E, F, heads)
    data = dict(d)
    for n_ in ("q", "k", "v", "att", "p", "y"):
        data[n_] = np.zeros(sh[n_], np.float32)
    diff = {n_: np.zeros(sh[n_], np.float32) for n_ in ("x", "q", "k", "v", "att", "p", "wo")}
    for n_ in ("wq", "wk", "wv"):
        diff[n_] = np.zeros((F, E), np.float32)
    diff["y"] = dyh
    am, keepm = hp.mhsa_args(pkg, data, diff, L, E, F, heads)
    olib = orc.load()
    f_fw = 4 * 2.0 * F * E * L + heads * 2 * 2.0 * L * L * (F // heads)
    add("mhsa L197 E192 3x64 FW N=1", "fp32", f_fw, lambda: olib.orc_mhsa_fw_fp32(ctypes.byref(am), 1))
    add("mhsa L197 E192 3x64 BW N=1", "fp32", 2 * f_fw, lambda: olib.orc_mhsa_bw_fp32(ctypes.byref(am), 1))
    return rows


def resnet_rows(pkg, lib, timed, torch, dev):
    """The ResNet-20-shaped training step, with and without normalisation layers."""
    rows = []
    tdt = {"fp32": torch.float32, "fp16": torch.float16}
    # config 5: ResNet-20 (CIFAR geometry) training step, fp16, batch 128, assembled from the entry points
    # (tests/resnet_step.py): with batch normalisation after every convolution, and without
    import resnet_step as rs
    ns, dt = 128, "fp16"
    convs, blocks, ncls = rs.resnet20_spec()
    macs, H = 3 * 16 * 9 * 32 * 32, 32
    for (n, ci, co, stride, proj) in blocks:
        Ho = H // stride
        macs += (ci * co * 9 + co * co * 9 + (ci * co if proj else 0)) * Ho * Ho
        H = Ho
    flops = 3 * 2.0 * ns * (macs + 64 * ncls)
    for norm, fused, stats, post, pre, head in ((True, True, False, False, False, False), (True, True, True, False, False, False),
                                                (True, True, True, True, False, False), (True, True, True, True, True, False),
                                                (True, True, True, True, True, True),
                                                (True, False, False, False, False, False), (False, False, False, False, False, False)):
        net = rs.ResNetStep(pkg, lib, torch, dt, ns, rs.init_weights(0x2E5E0, dt), 0.01, norm=norm, fused=fused, stats=stats,
                            post=post, pre=pre, head=head)
        net.x.copy_(torch.randn(ns, 3, 32, 32, device=dev).to(tdt[dt]))
        net.target.zero_()
        net.target[torch.arange(ns), torch.randint(0, 10, (ns,))] = 1
        ms = timed(lambda: net.step(update=True), 10, 3)
        rows.append({"workload": "resnet20 step%s FW+BW+SGD N=%d, %d launches"
                                 % ((" with batch norm" + (", element-wise layers fused into it" if fused else "") +
                                     (", its sums formed by the convolutions" if stats else "") +
                                     (" in both passes" if post else "") +
                                     (", applied inside the forward convolutions" if pre else "") +
                                     (", pooling + classifier + loss in one call" if head else "")) if norm
                                    else " (no norm)", ns, net.launches()),
                     "dtype": dt, "us": round(ms * 1e3, 1), "TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 3),
                     "samples/s": round(ns / (ms * 1e-3), 1)})
        if head:
            # the same step captured once into a HIP graph on a side stream and replayed (one submission per step
            # instead of 69 calls)
            import ctypes
            side = torch.cuda.Stream()
            lib.ptl_set_stream(ctypes.c_void_p(side.cuda_stream))
            try:
                with torch.cuda.stream(side):
                    net.step(update=True)
                    side.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        net.step(update=True)
                    ms = timed(graph.replay, 10, 3)
                rows.append({"workload": "resnet20 step with batch norm, all of the above, replayed as a HIP graph N=%d" % ns,
                             "dtype": dt, "us": round(ms * 1e3, 1), "TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 3),
                             "samples/s": round(ns / (ms * 1e-3), 1)})
                del graph
            finally:
                side.synchronize()
                lib.ptl_set_stream(None)
        del net
    return rows


def detail_table(pkg, lib, hp, to_dev, timed, check, torch, dev):
    """Per-step timings of the other BASELINE shapes: batch-1 latency and batched mode."""
    import ctypes
    rows = []

    def add(name, dt, ms, flops, nbytes):
        tf = flops / (ms * 1e-3) / 1e12
        gbs = nbytes / (ms * 1e-3) / 1e9
        bound = min(PEAK[dt], flops / max(nbytes, 1) * HBM_GBS / 1e3)  # TFLOP/s
        rows.append({"workload": name, "dtype": dt, "us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 3),
                     "GB/s": round(gbs, 1), "bound_TFLOP/s": round(bound, 1), "frac_of_bound": round(tf / bound, 4)})

    def run3(prefix, dt, a, ns, name, flops, bytes3, iters):
        ref = ctypes.byref(a)
        for s, nb in zip(("fw", "wg", "ig"), bytes3):
            f = getattr(lib, "%s_%s_%s_batched" % (prefix, dt, s))
            ms = timed(lambda: check(f(ref, ns)), iters)
            add("%s %s N=%d" % (name, s.upper(), ns), dt, ms, flops, nb)

    es = {"fp32": 4, "fp16": 2}
    tdt = {"fp32": torch.float32, "fp16": torch.float16}

    # config 1: Conv2D 16->32, 32x32, 3x3, pad 1 (fp32 as named; fp16 beside it), batch 1 and 128
    for dt in ("fp32", "fp16"):
        for ns in (1, 128):
            Ci, Co, H, W, K = 16, 32, 32, 32, 3
            x = torch.rand(ns, Ci, H, W, device=dev).to(tdt[dt]) - 0.5
            w = torch.rand(Co, Ci, K, K, device=dev).to(tdt[dt]) - 0.5
            dy = torch.rand(ns, Co, H, W, device=dev).to(tdt[dt]) - 0.5
            y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
            a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, W, Co, K, K, H, W, (1, 1, 1, 1))
            flops = 2.0 * ns * Co * Ci * K * K * H * W
            nb = (x.numel() + w.numel() + y.numel()) * es[dt]
            run3("ptl_conv2d", dt, a, ns, "conv2d 16->32 32x32 k3 p1", flops, (nb, nb, nb), 200 if ns == 1 else 50)

    # ResNet-20 stage-3 conv (64->64, 8x8) and stage-1 conv (16->16, 32x32), fp16, batch 128
    for (Ci, Co, H) in ((16, 16, 32), (64, 64, 8)):
        ns, K, dt = 128, 3, "fp16"
        x = torch.rand(ns, Ci, H, H, device=dev).to(tdt[dt]) - 0.5
        w = torch.rand(Co, Ci, K, K, device=dev).to(tdt[dt]) - 0.5
        dy = torch.rand(ns, Co, H, H, device=dev).to(tdt[dt]) - 0.5
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
        flops = 2.0 * ns * Co * Ci * K * K * H * H
        nb = (x.numel() + w.numel() + y.numel()) * es[dt]
        run3("ptl_conv2d", dt, a, ns, "conv2d %d->%d %dx%d k3 p1" % (Ci, Co, H, H), flops, (nb, nb, nb), 50)

    # config 2: Linear 1024x1024, batch 1 (both types) and 512 (fp32; fp16 is the headline)
    for dt, ns in (("fp32", 1), ("fp16", 1), ("fp32", 512), ("fp16", 8192)):
        n = 1024
        x = (torch.randn(ns, n, device=dev) / 32).to(tdt[dt])
        w = (torch.randn(n, n, device=dev) / 32).to(tdt[dt])
        dy = (torch.rand(ns, n, device=dev) - 0.5).to(tdt[dt])
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        a, keep = hp.linear_args(pkg, x, dx, w, dw, y, dy, n, n)
        flops = 2.0 * ns * n * n
        nb = (n * n + 2 * ns * n) * es[dt]
        run3("ptl_linear", dt, a, ns, "linear 1024x1024", flops, (nb, nb, nb), 200 if ns <= 512 else 20)

    # the same GEMM kernels on large plain products (the mm entry point): how far the tiles carry once launch and
    # first-trip latencies are amortised
    for dt, (N, M, K) in (("fp16", (4096, 4096, 4096)), ("fp32", (4096, 4096, 2048))):
        A = (torch.randn(N, K, device=dev) / 8).to(tdt[dt])
        Bm = (torch.randn(M, K, device=dev) / 8).to(tdt[dt])
        Cm = torch.zeros(N, M, device=dev, dtype=tdt[dt])
        f = lib.ptl_mm_fp16 if dt == "fp16" else lib.ptl_mm_fp32
        margs = [ctypes.c_void_p(A.data_ptr()), ctypes.c_void_p(Bm.data_ptr()), ctypes.c_void_p(Cm.data_ptr()), N, M, K, 1]
        ms = timed(lambda: check(f(*margs)), 10)
        add("mm %dx%dx%d (B transposed)" % (N, M, K), dt, ms, 2.0 * N * M * K, (N * K + M * K + N * M) * es[dt])
        del A, Bm, Cm

    # config 3: depthwise 3x3 on 64x56x56 (pre-padded 58x58) and pointwise 64->128, fp16, batch 1 and 64
    for ns in (1, 64):
        dt = "fp16"
        C, Hp, Ho, K = 64, 58, 56, 3
        x = (torch.rand(ns, C, Hp, Hp, device=dev) - 0.5).to(tdt[dt])
        w = (torch.rand(C, K, K, device=dev) - 0.5).to(tdt[dt])
        dy = (torch.rand(ns, C, Ho, Ho, device=dev) - 0.5).to(tdt[dt])
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        a, keep = hp.dw_args(pkg, dt, x, dx, w, dw, y, dy, C, Hp, Hp, K, K, Ho, Ho)
        flops = 2.0 * ns * C * K * K * Ho * Ho
        nb = (x.numel() + y.numel() + w.numel()) * 2
        run3("ptl_conv_dw", dt, a, ns, "depthwise 3x3 64x56x56", flops, (nb, nb, nb), 100 if ns == 1 else 30)
        Ci, Co, H = 64, 128, 56
        x = (torch.rand(ns, Ci, H * H, device=dev) - 0.5).to(tdt[dt])
        w = (torch.rand(Co, Ci, device=dev) - 0.5).to(tdt[dt])
        dy = (torch.rand(ns, Co, H * H, device=dev) - 0.5).to(tdt[dt])
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        a, keep = hp.pw_args(pkg, x, dx, w, dw, y, dy, Ci, Co, H, H)
        flops = 2.0 * ns * Co * Ci * H * H
        nb = (x.numel() + y.numel() + w.numel()) * 2
        run3("ptl_conv_pw", dt, a, ns, "pointwise 64->128 56x56", flops, (nb, nb, nb), 100 if ns == 1 else 30)

    # larger convolutions, fp16, batched (ResNet-18/50 style layers)
    # (the last three rows are a saturating sweep: the same kernels with enough tiles for several full rounds)
    # (128 -> 128 on 56x56: rows 57 wide, whose gradients take the resident-tile kernels since their input tiles share a ring)
    for (ns, Ci, Co, H) in ((256, 32, 64, 56), (128, 64, 64, 56), (64, 128, 128, 56), (128, 128, 128, 28),
                            (128, 256, 256, 14), (512, 128, 128, 28), (256, 256, 256, 28), (256, 512, 512, 14)):
        K, dt = 3, "fp16"
        x = torch.rand(ns, Ci, H, H, device=dev).to(tdt[dt]) - 0.5
        w = torch.rand(Co, Ci, K, K, device=dev).to(tdt[dt]) - 0.5
        dy = torch.rand(ns, Co, H, H, device=dev).to(tdt[dt]) - 0.5
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
        flops = 2.0 * ns * Co * Ci * K * K * H * H
        nb = (x.numel() + w.numel() + y.numel()) * es[dt]
        run3("ptl_conv2d", dt, a, ns, "conv2d %d->%d %dx%d k3 p1" % (Ci, Co, H, H), flops, (nb, nb, nb), 10)
        # weight + input gradient in one call (the two kernels share the blocked copy of the output gradient)
        ref = ctypes.byref(a)
        ms = timed(lambda: check(lib.ptl_conv2d_fp16_bw_batched(ref, ns)), 10)
        add("conv2d %d->%d %dx%d k3 p1 WG+IG in one call N=%d" % (Ci, Co, H, H, ns), dt, ms, 2 * flops, 2 * nb)
        # the same two calls reading the blocked copy of the input that the forward call left in a caller-owned buffer
        nbytes = lib.ptl_conv2d_fp16_cache_bytes(ref, ns)
        if nbytes:
            kept = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            cache = pkg.ConvCache()
            cache.buf, cache.bytes = kept.data_ptr(), nbytes
            check(lib.ptl_conv2d_fp16_fw_batched_cached(ref, ns, ctypes.byref(cache)))
            if cache.valid:
                ms = timed(lambda: check(lib.ptl_conv2d_fp16_wg_batched_cached(ref, ns, ctypes.byref(cache))), 10)
                add("conv2d %d->%d %dx%d k3 p1 WG, input copy kept by FW N=%d" % (Ci, Co, H, H, ns), dt, ms, flops, nb)
                ms = timed(lambda: check(lib.ptl_conv2d_fp16_bw_batched_cached(ref, ns, ctypes.byref(cache))), 10)
                add("conv2d %d->%d %dx%d k3 p1 WG+IG in one call, input copy kept by FW N=%d" % (Ci, Co, H, H, ns), dt,
                    ms, 2 * flops, 2 * nb)
                # layers in a row: the forward kernel also writes its output as the blocked copy the next layer reads
                # (timed here with the layer itself as that next layer: same channels in and out), and the forward call
                # of a layer that was handed such a copy
                if Ci == Co:
                    nxt = torch.empty(nbytes, dtype=torch.uint8, device=dev)
                    oc = pkg.ConvCache()
                    oc.buf, oc.bytes = nxt.data_ptr(), nbytes
                    check(lib.ptl_conv2d_fp16_cache_prepare(ref, ns, ctypes.byref(oc)))
                    ms = timed(lambda: check(lib.ptl_conv2d_fp16_fw_batched_chained(ref, ns, None, ctypes.byref(oc))), 10)
                    if oc.valid:
                        add("conv2d %d->%d %dx%d k3 p1 FW writing the next layer's input copy N=%d" % (Ci, Co, H, H, ns),
                            dt, ms, flops, nb)
                    ms = timed(lambda: check(lib.ptl_conv2d_fp16_fw_batched_chained(ref, ns, ctypes.byref(cache), None)), 10)
                    add("conv2d %d->%d %dx%d k3 p1 FW, input copy left by the layer before N=%d" % (Ci, Co, H, H, ns), dt,
                        ms, flops, nb)
                    ms = timed(lambda: check(lib.ptl_conv2d_fp16_fw_batched_chained(ref, ns, ctypes.byref(cache),
                                                                                     ctypes.byref(oc))), 10)
                    add("conv2d %d->%d %dx%d k3 p1 FW, copy in and copy out N=%d" % (Ci, Co, H, H, ns), dt, ms, flops, nb)
                    del nxt
                    # two such layers in a row, forward and backward: plain calls against the copies handed on and kept
                    if (ns, Ci, H) in ((256, 256, 28), (512, 128, 28)):
                        y2, dx2, dw2 = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
                        a2, keep2 = hp.conv2d_args(pkg, y, dx2, w, dw2, y2, dy, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
                        a1, keep1 = hp.conv2d_args(pkg, x, dx, w, dw, y, dx2, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1))
                        r1, r2 = ctypes.byref(a1), ctypes.byref(a2)

                        def plain_pair():
                            check(lib.ptl_conv2d_fp16_fw_batched(r1, ns))
                            check(lib.ptl_conv2d_fp16_fw_batched(r2, ns))
                            check(lib.ptl_conv2d_fp16_bw_batched(r2, ns))
                            check(lib.ptl_conv2d_fp16_bw_batched(r1, ns))

                        k1 = torch.empty(nbytes, dtype=torch.uint8, device=dev)
                        k2 = torch.empty(nbytes, dtype=torch.uint8, device=dev)
                        c1, c2 = pkg.ConvCache(), pkg.ConvCache()
                        c1.buf, c1.bytes = k1.data_ptr(), nbytes
                        c2.buf, c2.bytes = k2.data_ptr(), nbytes
                        check(lib.ptl_conv2d_fp16_cache_prepare(r2, ns, ctypes.byref(c2)))

                        def chained_pair():
                            c1.valid = 0
                            check(lib.ptl_conv2d_fp16_fw_batched_chained(r1, ns, ctypes.byref(c1), ctypes.byref(c2)))
                            check(lib.ptl_conv2d_fp16_fw_batched_chained(r2, ns, ctypes.byref(c2), None))
                            check(lib.ptl_conv2d_fp16_bw_batched_cached(r2, ns, ctypes.byref(c2)))
                            check(lib.ptl_conv2d_fp16_bw_batched_cached(r1, ns, ctypes.byref(c1)))

                        ms = timed(plain_pair, 5)
                        add("conv2d %d->%d %dx%d k3 p1 two layers in a row, FW + WG + IG, plain calls N=%d" % (Ci, Co, H, H, ns),
                            dt, ms, 6 * flops, 6 * nb)
                        ms = timed(chained_pair, 5)
                        add("conv2d %d->%d %dx%d k3 p1 two layers in a row, FW + WG + IG, copies handed on and kept N=%d"
                            % (Ci, Co, H, H, ns), dt, ms, 6 * flops, 6 * nb)
                        del k1, k2, y2, dx2, dw2
            del kept
        del x, w, dy, y, dx, dw

    # the same wide layers with channel-minor (HWC) tensors: X[b][h][w][ci], W[co][kh][kw][ci], Y[b][h][w][co]
    for (ns, Ci, Co, H) in ((128, 64, 64, 56), (128, 128, 128, 28), (128, 256, 256, 14)):
        K, dt = 3, "fp16"
        x = torch.rand(ns, H, H, Ci, device=dev).to(tdt[dt]) - 0.5
        w = torch.rand(Co, K, K, Ci, device=dev).to(tdt[dt]) - 0.5
        dy = torch.rand(ns, H, H, Co, device=dev).to(tdt[dt]) - 0.5
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        a, keep = hp.conv2d_args(pkg, x, dx, w, dw, y, dy, Ci, H, H, Co, K, K, H, H, (1, 1, 1, 1), (1, 1), 1)
        flops = 2.0 * ns * Co * Ci * K * K * H * H
        nb = (x.numel() + w.numel() + y.numel()) * es[dt]
        run3("ptl_conv2d", dt, a, ns, "conv2d HWC %d->%d %dx%d k3 p1" % (Ci, Co, H, H), flops, (nb, nb, nb), 10)
        del x, w, dy, y, dx, dw

    # config 4: multi-head self-attention step, fp32, L=197 E=192, 3 heads of 64, batch 1 and 32
    import numpy as np
    L, E, F, heads = 197, 192, 192, 3
    for ns in (1, 32):
        sh = hp.mhsa_shapes(ns, L, E, F, heads)
        d, dyh = hp.mhsa_inputs(0xC0DE0004, ns, L, E, F, heads)
        data = {n: to_dev(v) for n, v in d.items()}
        for n in ("q", "k", "v", "att", "p", "y"):
            data[n] = torch.zeros(sh[n], device=dev)
        diff = {n: torch.zeros(sh[n], device=dev) for n in ("x", "q", "k", "v", "att", "p", "wo")}
        for n in ("wq", "wk", "wv"):
            diff[n] = torch.zeros((F, E), device=dev)
        diff["y"] = to_dev(dyh)
        a, keep = hp.mhsa_args(pkg, data, diff, L, E, F, heads)
        ref = ctypes.byref(a)
        f_fw = ns * (4 * 2.0 * F * E * L + heads * 2 * 2.0 * L * L * (F // heads))
        act = ns * (2 * E * L + 4 * F * L + heads * L * L) * 4 + 4 * E * F * 4  # every tensor of the step once
        ms = timed(lambda: check(lib.ptl_mhsa_fp32_fw_batched(ref, ns)), 50)
        add("mhsa L197 E192 3x64 FW N=%d" % ns, "fp32", ms, f_fw, act)
        ms = timed(lambda: check(lib.ptl_mhsa_fp32_bw_batched(ref, ns)), 50)
        add("mhsa L197 E192 3x64 BW N=%d" % ns, "fp32", ms, 2 * f_fw, 2 * act)

    rows += helper_rows(pkg, lib, hp, timed, torch, dev)
    rows += resnet_rows(pkg, lib, timed, torch, dev)
    rows += power_rows(pkg, lib, hp, check, torch, dev)
    return rows


def helper_rows(pkg, lib, hp, timed, torch, dev):
    """The index-permutation and streaming helpers on tensors of 64 MiB and more, priced against HBM: GB/s of the
    bytes each must read plus the bytes it must write (the layout change is two passes by definition: transpose
    into the caller's buffer, copy back)."""
    import ctypes
    rows = []
    tdt = {"fp32": torch.float32, "fp16": torch.float16}
    es = {"fp32": 4, "fp16": 2}

    def add(name, dt, ms, nbytes):
        gbs = nbytes / (ms * 1e-3) / 1e9
        rows.append({"workload": name, "dtype": dt, "us": round(ms * 1e3, 2), "GB/s": round(gbs, 1),
                     "bound_GB/s": HBM_GBS, "frac_of_bound": round(gbs / HBM_GBS, 4)})

    def void_call(name, a):
        f = getattr(lib, name)
        ref = ctypes.byref(a)

        def go():
            f(ref)
            if lib.ptl_last_status() != 0:
                raise RuntimeError(lib.ptl_last_error().decode())
        return go

    for dt, (N, M) in (("fp16", (8192, 4096)), ("fp32", (4096, 4096))):
        sfx = "" if dt == "fp32" else "_fp16"
        src = torch.rand(N, M, device=dev).to(tdt[dt])
        dst = torch.zeros(M, N, device=dev, dtype=tdt[dt])
        a = pkg.TranspArgs()
        a.in_matrix, a.out_matrix, a.N, a.M = src.data_ptr(), dst.data_ptr(), N, M
        ms = timed(void_call("transpose_matrix" + sfx, a), 20)
        add("transpose_matrix %dx%d" % (N, M), dt, ms, 2 * N * M * es[dt])
        c = pkg.CopyArgs()
        c.from_, c.to, c.size = src.data_ptr(), dst.data_ptr(), N * M
        ms = timed(void_call("copy" + sfx, c), 20)
        add("copy %d elements" % (N * M), dt, ms, 2 * N * M * es[dt])
        del src, dst
    # layout change CHW -> HWC of a 256 x 256 x 512 tensor (64 MiB in fp16): transpose + copy back = 4 x the tensor
    C, H, W, dt = 256, 256, 512, "fp16"
    t = torch.rand(C, H, W, device=dev).to(tdt[dt])
    buf = torch.zeros(C * H * W, device=dev, dtype=tdt[dt])
    b = pkg.blob(t, None, C, H, W)
    la = pkg.LayoutArgs()
    la.tensor, la.transp_buffer, la.transpose_data, la.transpose_grad = hp.ptr(b), buf.data_ptr(), 1, 0
    ms = timed(void_call("CHW_to_HWC_fp16", la), 10)
    add("CHW_to_HWC %dx%dx%d (two passes)" % (C, H, W), dt, ms, 4 * C * H * W * es[dt])
    ms = timed(void_call("HWC_to_CHW_fp16", la), 10)
    add("HWC_to_CHW %dx%dx%d (two passes)" % (C, H, W), dt, ms, 4 * C * H * W * es[dt])
    del t, buf
    # weight block transpose, 2048 x 2048 channels, 3x3 (72 MiB in fp16), both layouts
    Ci = Co = 2048
    for hwc in (0, 1):
        w = torch.rand(Co * Ci * 9, device=dev).to(tdt[dt])
        bt = torch.zeros_like(w)
        g = pkg.BlocktranspArgs()
        g.weights, g.bt_weights, g.Cin, g.Cout, g.Hk, g.Wk, g.HWC = w.data_ptr(), bt.data_ptr(), Ci, Co, 3, 3, hwc
        ms = timed(void_call("pulp_blocktransp_fp16", g), 10)
        add("blocktranspose %dx%dx3x3 %s" % (Co, Ci, "HWC" if hwc else "CHW"), dt, ms, 2 * w.numel() * es[dt])
        del w, bt
    # im2row of a 64 x 224 x 224 input, 3x3, pad 1 (patch matrix 50176 x 576), fp32 (110 MiB) and fp16
    for dt in ("fp32", "fp16"):
        Ci, H, K = 64, 224, 3
        x = torch.rand(Ci, H, H, device=dev).to(tdt[dt])
        buf = torch.zeros(H * H * Ci * K * K, device=dev, dtype=tdt[dt])
        bi, bw, bo = pkg.blob(x, None, Ci, H, H), pkg.blob(None, None, Ci, K, K), pkg.blob(None, None, 1, H, H)
        a = pkg.Im2colArgs()
        a.input, a.c, a.output, a.pBuffer = hp.ptr(bi), hp.ptr(bw), hp.ptr(bo), buf.data_ptr()
        a.Lpad = a.Rpad = a.Upad = a.Dpad = 1
        a.stride_h = a.stride_w = 1
        ms = timed(void_call("pulp_im2row_" + dt, a), 10)
        add("im2row 64x224x224 k3 p1", dt, ms, (x.numel() + buf.numel()) * es[dt])
        if dt == "fp16":  # the column-major patch matrix of the same input
            ms = timed(void_call("pulp_im2col_" + dt, a), 10)
            add("im2col 64x224x224 k3 p1", dt, ms, (x.numel() + buf.numel()) * es[dt])
        del x, buf
    # pad_tensor 256 x 360 x 360 by one on every side (63 MiB -> 64 MiB in fp16)
    C, H, dt = 256, 360, "fp16"
    srct = torch.rand(C, H, H, device=dev).to(tdt[dt])
    dstt = torch.zeros(C, H + 2, H + 2, device=dev, dtype=tdt[dt])
    pa = pkg.PadArgs()
    pa.source, pa.dest, pa.C, pa.H, pa.W = srct.data_ptr(), dstt.data_ptr(), C, H, H
    pa.T_RPAD = pa.T_LPAD = pa.T_UPAD = pa.T_DPAD = 1
    ms = timed(void_call("pad_tensor_fp16", pa), 10)
    add("pad_tensor %dx%dx%d pad 1" % (C, H, H), dt, ms, (srct.numel() + dstt.numel()) * es[dt])
    return rows


if __name__ == "__main__":
    main()
