"""Headline benchmark: fp32 convolution throughput (fprop + dgrad + wgrad) on one
MI355X, on the ResNet-style shape input NHWC [256,56,56,64], 64 filters 3x3,
stride 1, "same" padding.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one batch: Conv_Layer's three
contractions (fprop with fused bias, dgrad, wgrad with dbias) through the C ABI,
inputs already resident in HBM.  Prints ONE JSON line.  `value` is the
algorithmic TFLOP/s of the whole step (3 * 2*M*N*K flops / step time); the
per-direction figures, the bf16 variant and the training-step images/sec are
reported under "extra".  The CPU baseline is the NumPy einsum oracle timed on a
bounded sample (a smaller batch of the same layer) on this machine's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "aether-ml_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import numpy as np

FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0


def conv_flops(S, Ho, Wo, fH, fW, C, D):
    return 2.0 * S * Ho * Wo * fH * fW * C * D


def time_loop(fn, steps, warmup):
    """Average ms per call from HIP events on the library's stream."""
    from aether import _lib
    for _ in range(warmup):
        fn()
    _lib.sync()
    e0, e1 = _lib.Event(), _lib.Event()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    return e0.elapsed_ms(e1) / steps


COUNTERS = os.path.join(ROOT, "profiles", "conv_f32_resnet3x3_256x56x56x64.counters.json")


def sources_digest():
    """SHA-256 over the kernel sources (aether-ml_amd/csrc, in name order): what a counter summary is stamped
    with, so that a later run can tell whether the kernels it times are the ones the counters saw."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "aether-ml_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".h", ".hip")):
            h.update(name.encode())
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def counter_traffic(kernel):
    """(bytes, source): HBM/fabric bytes per launch of `kernel` from the summary that the last FETCH_SIZE /
    WRITE_SIZE counter runs of this benchmark left under profiles/ (bench_counters.py writes it, scaled by what
    the same counters read for a plain copy of known size), and where that figure comes from: the file, when it
    was measured, the digest of the kernel sources it was measured on and whether that is the digest of the
    sources of this run.  The figure is NOT measured in this run (counters need the profiler); a summary taken on
    other sources is reported as stale, with a warning.  (None, None) when the file or the kernel is missing."""
    try:
        with open(COUNTERS) as f:
            doc = json.load(f)
        traffic = float(doc["kernels"][kernel]["traffic_bytes"])
    except (OSError, KeyError, ValueError, TypeError):
        return None, None
    stamp = doc.get("measured", {})
    now = sources_digest()
    source = {"file": os.path.relpath(COUNTERS, ROOT), "measured_on": stamp.get("date"),
              "sources_digest": stamp.get("sources_digest"), "this_run_sources_digest": now,
              "same_sources": stamp.get("sources_digest") == now,
              "how": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this benchmark, summarised by bench_counters.py"}
    if not source["same_sources"]:
        print("bench.py: roofline.traffic comes from counters measured on other kernel sources (%s, now %s): "
              "re-run the counter passes (bench_counters.py)" % (source["sources_digest"], now), file=sys.stderr)
    return traffic, source


def cpu_baseline(S_small, H, W, C, D):
    """NumPy einsum oracle (single-threaded by construction) on a reduced batch."""
    from oracle import oracle as O
    r = np.random.RandomState(1)
    x = r.randn(S_small, H, W, C).astype(np.float32)
    w = (r.randn(3, 3, C, D) * np.sqrt(2.0 / (9 * C))).astype(np.float32)
    b = np.zeros(D, np.float32)
    dy = r.randn(S_small, H, W, D).astype(np.float32)
    t0 = time.perf_counter()
    O.conv_fprop(x, w, b, (1, 1), "same")
    t1 = time.perf_counter()
    O.conv_dgrad(dy, w, (H, W), (1, 1), "same")
    t2 = time.perf_counter()
    O.conv_wgrad(x, dy, (3, 3), (1, 1), "same")
    O.conv_dbias(dy)
    t3 = time.perf_counter()
    fl = conv_flops(S_small, H, W, 3, 3, C, D)
    return {
        "value": 3 * fl / (t3 - t0) / 1e12,
        "unit": "TFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample_batch": S_small,
        "config_batch": 256,
        "scaled_from": "time is linear in the batch: the figure is flops of the sample / seconds of the sample",
        "sample": "same layer, batch %d instead of 256 (fprop %.2fs, dgrad %.2fs, wgrad %.2fs); np.einsum is single-threaded; host has %d cores"
                  % (S_small, t1 - t0, t2 - t1, t3 - t2, os.cpu_count()),
        "per_direction_gflops": {"fprop": fl / (t1 - t0) / 1e9, "dgrad": fl / (t2 - t1) / 1e9,
                                 "wgrad": fl / (t3 - t2) / 1e9},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the bf16 / train-step extras")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch relu_fwd_kernel with alpha=1 (a plain copy) over 64 Mi floats three times: "
                         "256 MiB read + 256 MiB written per launch, the yardstick for FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from aether import _lib
    from aether.tensor import DeviceTensor
    L = _lib.lib()
    info = _lib.device_info()

    S, H, W, C, D = 256, 56, 56, 64, 64
    dims = (S, H, W, C, D, 3, 3, 1, 1, 1, 1)
    np.random.seed(0)
    x_h = np.random.randn(S, H, W, C).astype(np.float32)
    w_h = (np.random.randn(3, 3, C, D).astype(np.float32) * np.float32(np.sqrt(2.0 / (9 * C))))
    dy_h = np.random.randn(S, H, W, D).astype(np.float32)
    x, w, dy = (DeviceTensor.from_numpy(a) for a in (x_h, w_h, dy_h))
    bias = DeviceTensor.zeros(D)
    y, dx = DeviceTensor((S, H, W, D)), DeviceTensor((S, H, W, C))
    dw, db = DeviceTensor((3, 3, C, D)), DeviceTensor(D)
    del x_h, dy_h

    def fprop():
        _lib.check(L.aeth_conv_fprop_f32(x.ptr, w.ptr, bias.ptr, y.ptr, *dims))

    def dgrad():
        _lib.check(L.aeth_conv_dgrad_f32(dy.ptr, w.ptr, dx.ptr, *dims))

    def wgrad():
        _lib.check(L.aeth_conv_wgrad_f32(x.ptr, dy.ptr, dw.ptr, db.ptr, *dims))

    def step():
        fprop()
        wgrad()
        dgrad()

    fl = conv_flops(S, H, W, 3, 3, C, D)

    if args.copy_probe:
        n = 64 * 1024 * 1024
        src, dst = DeviceTensor.zeros(n), DeviceTensor(n)
        for _ in range(3):
            _lib.check(L.aeth_relu_fwd_f32(src.ptr, dst.ptr, 1.0, n))
        _lib.sync()
        del src, dst

    # ---- each direction alone in a loop (reported under extra, not the roofline) ----
    # Before the timed steps: 20 steps and some 70 launches (60 ms) also bring the device to the clocks it keeps
    # under load; timed right after 5 warm-up steps alone, the first steps of the region ran 5 % slower
    # (1.411 against 1.334 ms per step in alternating runs on one box).
    for _ in range(20):
        step()
    per = {}
    for name, fn in (("fprop", fprop), ("dgrad", dgrad), ("wgrad", wgrad)):
        ms = time_loop(fn, args.steps, 2)
        per[name] = {"ms": ms, "tflops": fl / (ms * 1e-3) / 1e12,
                     "frac_fp32_mfma_peak": fl / (ms * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS}
    # ---- the timed region: exactly K steps between two synchronisations --------
    # Events between the directions of every step give each kernel's duration INSIDE the
    # step the headline is quoted on.
    for _ in range(args.warmup):
        step()
    _lib.sync()
    marks = [[_lib.Event() for _ in range(4)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    e0, e1 = _lib.Event(), _lib.Event()
    e0.record()
    for k in range(args.steps):
        m = marks[k]
        m[0].record()
        fprop()
        m[1].record()
        wgrad()
        m[2].record()
        dgrad()
        m[3].record()
    e1.record()
    _lib.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = e0.elapsed_ms(e1) / args.steps
    ms_per_step = max(ms_per_step, 0.0)
    value = 3 * fl / (ms_per_step * 1e-3) / 1e12
    in_step = {}
    for i, name in enumerate(("fprop", "wgrad", "dgrad")):
        ms = sum(m[i].elapsed_ms(m[i + 1]) for m in marks) / args.steps
        in_step[name] = {"ms": ms, "tflops": fl / (ms * 1e-3) / 1e12,
                         "frac_fp32_mfma_peak": fl / (ms * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS}

    # The dominant kernel is the one with the largest share of the step: gather_classes_f32 runs twice per step (fprop
    # and dgrad, each cut into the nine parts that see the same taps inside the image, the parts in one launch whose
    # workgroups run the body of gather_gemm_dma; both read the filter in place: no packing launch), wgrad_halo_f32
    # once (its interval also holds the reduction of its split sums, a few us).  `achieved` = algorithmic flops per
    # launch / the kernel's average duration inside the timed steps.  The slowest direction is reported beside it.
    gather_ms = 0.5 * (in_step["fprop"]["ms"] + in_step["dgrad"]["ms"])
    share = {"gather_classes_f32": 2 * gather_ms, "wgrad_halo_f32": in_step["wgrad"]["ms"]}
    kernel = max(share, key=share.get)
    kernel_ms = gather_ms if kernel == "gather_classes_f32" else in_step["wgrad"]["ms"]
    achieved = fl / (kernel_ms * 1e-3) / 1e12
    slowest = min(in_step, key=lambda k: in_step[k]["tflops"])
    traffic, traffic_source = counter_traffic(kernel)
    roofline = {
        "bound": "mfma",
        "kernel": kernel,
        "achieved": achieved,
        "peak": FP32_MFMA_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
        "traffic": traffic,
        "traffic_source": traffic_source,
        "launch_ms_in_step": kernel_ms,
        "share_of_step": share[kernel] / sum(share.values()),
        "slowest_direction": {"direction": slowest, "tflops": in_step[slowest]["tflops"],
                              "frac": in_step[slowest]["frac_fp32_mfma_peak"]},
        "algorithmic_flops_per_launch": fl,
        "algorithmic_bytes_per_launch": 4.0 * (2 * S * H * W * C + 9 * C * D + D),
    }

    extra = {"per_direction_fp32_in_step": in_step, "per_direction_fp32_alone_in_a_loop": per,
             "wall_ms_per_step": wall_ms,
             "device": {k: info[k] for k in ("arch", "cus", "clock_mhz")}}
    if not args.no_extra:
        try:
            import bench_extra
            extra.update(bench_extra.run(args.steps, args.warmup))
        except Exception as e:   # extras never hide the headline number
            extra["extra_error"] = "%s: %s" % (type(e).__name__, e)

    out = {
        "metric": "conv TFLOP/s (fprop+dgrad+wgrad), fp32 MFMA",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Conv_Layer fwd+bwd, input NHWC [256,56,56,64], 64 filters 3x3 stride 1 same pad, "
                               "He-normal weights, N(0,1) input and upstream gradient, seed 0",
                   "frac_fp32_mfma_peak": value / FP32_MFMA_PEAK_TFLOPS},
        "roofline": roofline,
        "extra": extra,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(128, H, W, C, D)
        if not args.no_extra:
            try:
                import bench_extra
                extra["cpu_other_configs"] = bench_extra.cpu_table()
            except Exception as e:
                extra["cpu_other_error"] = "%s: %s" % (type(e).__name__, e)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
