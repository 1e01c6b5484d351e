"""Secondary measurements printed under "extra" by bench.py: every convolution
shape of the benchmark list in fp32 (and bf16-input where the list asks for it),
per direction, and the three-block CNN training step in images/sec."""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "aether-ml_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

FP32_PEAK = 157.3
BF16_PEAK = 2500.0
HBM_GBS = 8000.0

# name, S, H, W, C, D, f, stride, pad P, bf16 too?
SHAPES = [
    ("cfg1_32x32x3_to32", 128, 32, 32, 3, 32, 3, 1, 1, False),
    ("cfg2a_16x16x32_to64", 128, 16, 16, 32, 64, 3, 1, 1, False),
    ("cfg2b_8x8x64_to128", 128, 8, 8, 64, 128, 3, 1, 1, False),
    ("cfg4_56x56x64_to64", 256, 56, 56, 64, 64, 3, 1, 1, True),
    ("cfg4_1x1_64_to256", 256, 56, 56, 64, 256, 1, 1, 0, True),
    ("cfg5_28x28x128_to256_s2", 1024, 28, 28, 128, 256, 3, 2, 0, True),
]


def _time(fn, steps, warmup):
    """Average ms per call over `steps` calls, after at least `warmup` calls and
    40 ms of back-to-back work (so clocks have ramped after the host-side setup)."""
    from aether import _lib
    t0 = time.perf_counter()
    n = 0
    while n < warmup or time.perf_counter() - t0 < 0.04:
        fn()
        n += 1
        if n % 8 == 0:
            _lib.sync()
    _lib.sync()
    e0, e1 = _lib.Event(), _lib.Event()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    return e0.elapsed_ms(e1) / steps


def conv_table(steps, warmup, only=None):
    from aether import _lib
    from aether.tensor import DeviceTensor
    L = _lib.lib()
    rng = np.random.default_rng(0)
    out = {}
    for name, S, H, W, C, D, f, st, P, with_bf16 in SHAPES:
        if only is not None and name != only:
            continue
        Ho = (H + 2 * P - f) // st + 1
        Wo = (W + 2 * P - f) // st + 1
        dims = (S, H, W, C, D, f, f, st, st, P, P)
        x = DeviceTensor.from_numpy(rng.standard_normal((S, H, W, C), dtype=np.float32))
        w = DeviceTensor.from_numpy(rng.standard_normal((f, f, C, D), dtype=np.float32) *
                                    np.float32(np.sqrt(2.0 / (f * f * C))))
        dy = DeviceTensor.from_numpy(rng.standard_normal((S, Ho, Wo, D), dtype=np.float32))
        b = DeviceTensor.zeros(D)
        y, dx = DeviceTensor((S, Ho, Wo, D)), DeviceTensor((S, H, W, C))
        dw, db = DeviceTensor((f, f, C, D)), DeviceTensor(D)
        flops = 2.0 * S * Ho * Wo * f * f * C * D
        nx, ny, nw = S * H * W * C, S * Ho * Wo * D, f * f * C * D
        row = {"gflop_per_direction": flops / 1e9}
        calls = {
            "fprop": lambda: _lib.check(L.aeth_conv_fprop_f32(x.ptr, w.ptr, b.ptr, y.ptr, *dims)),
            "dgrad": lambda: _lib.check(L.aeth_conv_dgrad_f32(dy.ptr, w.ptr, dx.ptr, *dims)),
            "wgrad": lambda: _lib.check(L.aeth_conv_wgrad_f32(x.ptr, dy.ptr, dw.ptr, db.ptr, *dims)),
        }
        byts = {"fprop": 4 * (nx + nw + D + ny), "dgrad": 4 * (ny + nw + nx), "wgrad": 4 * (nx + ny + nw + D)}
        for k, fn in calls.items():
            ms = _time(fn, steps, warmup)
            row["f32_" + k] = {"ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 3),
                               "frac_mfma_peak": round(flops / ms / 1e9 / FP32_PEAK, 4),
                               "frac_hbm_peak": round(byts[k] / ms / 1e6 / HBM_GBS, 4)}
        if with_bf16:
            x16, w16, dy16 = (DeviceTensor(t.shape, np.uint16) for t in (x, w, dy))
            for src, dst in ((x, x16), (w, w16), (dy, dy16)):
                _lib.check(L.aeth_cast_f32_to_bf16(src.ptr, dst.ptr, src.size))
            calls = {
                "fprop": lambda: _lib.check(L.aeth_conv_fprop_bf16(x16.ptr, w16.ptr, b.ptr, y.ptr, *dims)),
                "dgrad": lambda: _lib.check(L.aeth_conv_dgrad_bf16(dy16.ptr, w16.ptr, dx.ptr, *dims)),
                "wgrad": lambda: _lib.check(L.aeth_conv_wgrad_bf16(x16.ptr, dy16.ptr, dw.ptr, db.ptr, *dims)),
            }
            byts = {"fprop": 2 * (nx + nw) + 4 * (D + ny), "dgrad": 2 * (ny + nw) + 4 * nx,
                    "wgrad": 2 * (nx + ny) + 4 * (nw + D)}
            for k, fn in calls.items():
                ms = _time(fn, steps, warmup)
                row["bf16_" + k] = {"ms": round(ms, 5), "tflops": round(flops / ms / 1e9, 3),
                                    "frac_mfma_peak": round(flops / ms / 1e9 / BF16_PEAK, 4),
                                    "frac_hbm_peak": round(byts[k] / ms / 1e6 / HBM_GBS, 4)}
        out[name] = row
        del x, w, dy, y, dx
    return out


def build_cnn(aether):
    """Conv(32)-BN-ReLU-Pool, Conv(64)-BN-ReLU-Pool, Conv(128)-BN-ReLU-Pool, Flatten,
    Dense 2048->256, LeakyReLU(0.01), Dense 256->10, softmax CCE(ls 0.01), Adam 1e-3."""
    m = aether.Model()
    c, size = 3, 32
    for d in (32, 64, 128):
        m.add(aether.Conv_Layer((size, size, c), num_filters=d, filter_size=(3, 3), strides=(1, 1), padding="same"))
        m.add(aether.Batch_Norm())
        m.add(aether.ReLU())
        m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
        c, size = d, size // 2
    m.add(aether.Flatten())
    m.add(aether.Layer_Dense(size * size * 128, 256))
    m.add(aether.Leaky_ReLU(alpha=0.01))
    m.add(aether.Layer_Dense(256, 10))
    m.add(aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(label_smoothing=0.01),
          optimizer=aether.Optimizer_Adam(learning_rate=1e-3), accuracy=aether.Accuracy_Categorical())
    m.finalize()
    return m


def train_step(steps, warmup, eager_only=False):
    """`eager_only`: no recorded steps and no Model.train loops (a kernel trace of the step: the launches of an eager step
    are those a recording replays)."""
    import aether
    from aether import _lib
    np.random.seed(0)
    X = aether.DeviceTensor.from_numpy(np.random.rand(128, 32, 32, 3).astype(np.float32))
    y = np.random.randint(0, 10, 128)

    def timed(model):
        model.loss.new_pass()
        model.accuracy.new_pass()
        for _ in range(warmup):
            model.train_step(X, y)
        _lib.sync()
        times = []
        for _ in range(steps):
            t0 = time.perf_counter()
            loss, data_loss, reg, acc = model.train_step(X, y)
            _lib.sync()
            times.append(time.perf_counter() - t0)
        return float(np.median(times)), float(loss)

    np.random.seed(0)
    med, loss = timed(build_cnn(aether))
    if eager_only:
        return {"ms_per_step_median": med * 1e3, "images_per_sec": 128.0 / med, "batch": 128, "last_loss": loss}
    np.random.seed(0)
    recorded = build_cnn(aether)
    recorded.record_steps(True)
    med_rec, loss_rec = timed(recorded)

    def train_loop(record):
        """Model.train over a data set that lives on the device (64 batches of 128, 3 epochs after one to settle):
        seconds of the whole call per step, printing every 100th step as the reference's scripts do."""
        import contextlib
        import io
        np.random.seed(1)
        Xs = aether.DeviceTensor.from_numpy(np.random.rand(64 * 128, 32, 32, 3).astype(np.float32))
        ys = np.random.randint(0, 10, 64 * 128)
        np.random.seed(0)
        model = build_cnn(aether)
        model.record_steps(record)
        with contextlib.redirect_stdout(io.StringIO()):
            model.train(Xs, ys, epochs=1, batch_size=128, print_every=100)
            _lib.sync()
            t0 = time.perf_counter()
            model.train(Xs, ys, epochs=3, batch_size=128, print_every=100)
            _lib.sync()
            dt = time.perf_counter() - t0
        return dt / (3 * 64)

    loop, loop_rec = train_loop(False), train_loop(True)
    return {"ms_per_step_median": med * 1e3, "images_per_sec": 128.0 / med, "batch": 128, "last_loss": loss,
            "train_loop": {"ms_per_step": loop * 1e3, "images_per_sec": 128.0 / loop,
                           "recorded_ms_per_step": loop_rec * 1e3, "recorded_images_per_sec": 128.0 / loop_rec,
                           "note": "Model.train(X, y, epochs=3, batch_size=128, print_every=100) on 8192 images resident in HBM: "
                                   "wall time of the call per step; the host reads a step's loss and predictions while the "
                                   "next step runs, with steps launched kernel by kernel and with replayed ones"},
            "recorded_steps": {"ms_per_step_median": med_rec * 1e3, "images_per_sec": 128.0 / med_rec,
                               "last_loss": loss_rec,
                               "note": "Model.record_steps(True): the step replayed from a HIP graph, one host call"},
            "note": "forward + loss + accuracy + backward + Adam, batch resident in HBM, "
                    "includes the per-step scalar read-backs"}


def cpu_table():
    """The NumPy einsum oracle on the other benchmark configurations, one core: 1 warm-up +
    3 runs (median) for the small layers, one run of one training step of the three-block
    CNN, one run of a batch-16 sample of the stride-2 layer.  Seconds and GFLOP/s per
    direction, next to which the GPU figures of `conv_shapes` stand."""
    from oracle import oracle as O
    out = {"numpy": np.__version__, "host_cores": os.cpu_count(), "threads_used": 1}
    rng = np.random.RandomState(0)

    def layer(S, H, W, C, D, f, st, pad, runs):
        x = rng.randn(S, H, W, C).astype(np.float32)
        w = (rng.randn(f, f, C, D) * np.sqrt(2.0 / (f * f * C))).astype(np.float32)
        b = np.zeros(D, np.float32)
        y = O.conv_fprop(x, w, b, (st, st), pad)
        dy = rng.randn(*y.shape).astype(np.float32)
        flops = 2.0 * y.size * f * f * C
        res = {"batch": S}
        for name, fn in (("fprop", lambda: O.conv_fprop(x, w, b, (st, st), pad)),
                         ("dgrad", lambda: O.conv_dgrad(dy, w, (H, W), (st, st), pad)),
                         ("wgrad", lambda: (O.conv_wgrad(x, dy, (f, f), (st, st), pad), O.conv_dbias(dy)))):
            ts = []
            for _ in range(runs):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            sec = float(np.median(ts))
            res[name] = {"seconds": round(sec, 4), "gflops": round(flops / sec / 1e9, 2)}
        return res

    for name, S, H, W, C, D, f, st, P, _ in SHAPES[:3]:
        layer(S, H, W, C, D, f, st, "same", 1)                                   # warm-up
        out[name] = layer(S, H, W, C, D, f, st, "same", 3)
    out["cfg5_28x28x128_to256_s2"] = dict(layer(16, 28, 28, 128, 256, 3, 2, "valid", 1),
                                          note="batch 16 of 1024; time is linear in the batch")
    np.random.seed(0)
    X = np.random.rand(128, 32, 32, 3).astype(np.float32)
    y = np.random.randint(0, 10, 128)
    net = O.OracleCNN(O.make_cnn_params(dtype=np.float32), dtype=np.float32)
    t0 = time.perf_counter()
    net.step(X, y)
    sec = time.perf_counter() - t0
    out["train_step_cnn3"] = {"seconds_per_step": round(sec, 3), "images_per_sec": round(128.0 / sec, 2), "batch": 128}
    return out


def bf16_layer(steps, warmup):
    """Conv_Layer.forward + backward on bf16 inputs THROUGH THE LAYER on the headline shape, next
    to the sum of the three ABI calls: (a) a lone layer handed float32 tensors, which has to cast
    x and dy itself (two passes of 308 MB each); (b) the same layer fed by producers that leave
    bfloat16 copies beside their float32 outputs, as ReLU / the fused batch-norm block / batch
    norm's backward pass do inside a model, so that only the filter is cast."""
    import aether
    from aether import _lib
    from aether.tensor import DeviceTensor
    L = _lib.lib()
    S, H, W, C, D = 256, 56, 56, 64, 64
    rng = np.random.default_rng(0)
    x = DeviceTensor.from_numpy(rng.standard_normal((S, H, W, C), dtype=np.float32))
    dy = DeviceTensor.from_numpy(rng.standard_normal((S, H, W, D), dtype=np.float32))
    np.random.seed(0)
    layer = aether.Conv_Layer((H, W, C), num_filters=D, filter_size=(3, 3), strides=(1, 1), padding="same")
    layer.precision = "bf16"

    def step():
        layer.forward(x, True)
        layer.backward(dy)

    alone = _time(step, steps, warmup)
    for t in (x, dy):
        t._bf16 = DeviceTensor(t.shape, np.uint16)
        _lib.check(L.aeth_cast_f32_to_bf16(t.ptr, t._bf16.ptr, t.size))
    fed = _time(step, steps, warmup)
    x16, dy16, w16 = x._bf16, dy._bf16, layer._filter_bf16()
    dims = (S, H, W, C, D, 3, 3, 1, 1, 1, 1)
    y, dx, dw, db = layer.output, layer.dinputs, layer.dweights, layer.dbiases

    def abi():
        _lib.check(L.aeth_conv_fprop_bf16(x16.ptr, w16.ptr, layer.biases.ptr, y.ptr, *dims))
        _lib.check(L.aeth_conv_wgrad_bf16(x16.ptr, dy16.ptr, dw.ptr, db.ptr, *dims))
        _lib.check(L.aeth_conv_dgrad_bf16(dy16.ptr, w16.ptr, dx.ptr, *dims))

    calls = _time(abi, steps, warmup)
    cast = _time(lambda: _lib.check(L.aeth_cast_f32_to_bf16(x.ptr, x16.ptr, x.size)), steps, warmup)
    flops = 3 * 2.0 * S * H * W * 9 * C * D
    return {"shape": "Conv_Layer fwd+bwd, bf16 inputs, NHWC [256,56,56,64] -> 64 filters 3x3",
            "abi_calls_ms": round(calls, 4), "abi_calls_tflops": round(flops / calls / 1e9, 1),
            "layer_fed_by_producers_ms": round(fed, 4), "layer_fed_by_producers_tflops": round(flops / fed / 1e9, 1),
            "layer_alone_casting_x_and_dy_ms": round(alone, 4),
            "layer_alone_casting_x_and_dy_tflops": round(flops / alone / 1e9, 1),
            "cast_205MB_tensor_ms": round(cast, 4), "cast_tb_per_s": round(x.size * 6 / cast / 1e9, 2),
            "layer_over_abi": round(fed / calls, 3)}


def layer_kernels(steps, warmup):
    """The supporting kernels on the headline tensor, NHWC [256,56,56,64] fp32 (205.5 MB): ms per call and
    algorithmic bytes / time.  A call that is several launches (batch norm: partial sums, their reduction,
    the apply pass) is timed as a whole and priced with the bytes its passes must move."""
    import ctypes as C
    from aether import _lib
    from aether.tensor import DeviceTensor
    L = _lib.lib()
    S, H, W, Ch = 256, 56, 56, 64
    n = S * H * W * Ch
    rows = S * H * W
    rng = np.random.default_rng(0)
    x = DeviceTensor.from_numpy(rng.standard_normal((S, H, W, Ch), dtype=np.float32))
    dy = DeviceTensor.from_numpy(rng.standard_normal((S, H, W, Ch), dtype=np.float32))
    y, y2, y3 = (DeviceTensor((S, H, W, Ch)) for _ in range(3))
    gamma = DeviceTensor.from_numpy(np.ones(Ch, np.float32))
    rv = DeviceTensor.from_numpy(np.ones(Ch, np.float32))
    beta, rm, sm, si, dgamma, dbeta = (DeviceTensor.zeros(Ch) for _ in range(6))
    pooled = DeviceTensor((S, H // 2, W // 2, Ch))
    dpooled = DeviceTensor.from_numpy(rng.standard_normal((S, H // 2, W // 2, Ch), dtype=np.float32))
    idx = DeviceTensor((n // 16,))                          # one byte per pooled element
    f, i64 = C.c_float, C.c_int64
    fp = 4 * n                                              # bytes of one full-size tensor
    calls = [
        ("relu_fwd", 2 * fp, lambda: L.aeth_relu_fwd_f32(x.ptr, y.ptr, f(0.0), i64(n))),
        ("relu_bwd", 3 * fp, lambda: L.aeth_relu_bwd_f32(x.ptr, dy.ptr, y.ptr, f(0.0), i64(n))),
        ("bn_fwd_train (3 launches)", 3 * fp, lambda: L.aeth_bn_fwd_train_f32(
            x.ptr, gamma.ptr, beta.ptr, rm.ptr, rv.ptr, sm.ptr, si.ptr, y.ptr, rows, Ch, f(1e-5), f(0.9))),
        ("bn_bwd (3 launches)", 5 * fp, lambda: L.aeth_bn_bwd_f32(
            x.ptr, dy.ptr, gamma.ptr, sm.ptr, si.ptr, y.ptr, dgamma.ptr, dbeta.ptr, rows, Ch)),
        ("maxpool_fwd 2x2/2", fp + fp // 4 + n // 4, lambda: L.aeth_maxpool_fwd_f32(
            x.ptr, pooled.ptr, idx.ptr, S, H, W, Ch, 2, 2, 2, 2)),
        ("maxpool_bwd 2x2/2", fp + fp // 4 + n // 4, lambda: L.aeth_maxpool_bwd_f32(
            dpooled.ptr, idx.ptr, y.ptr, S, H, W, Ch, 2, 2, 2, 2)),
        ("avgpool_fwd 2x2/2", fp + fp // 4, lambda: L.aeth_avgpool_fwd_f32(x.ptr, pooled.ptr, S, H, W, Ch, 2, 2, 2, 2)),
        ("avgpool_bwd 2x2/2", fp + fp // 4, lambda: L.aeth_avgpool_bwd_f32(dpooled.ptr, y.ptr, S, H, W, Ch, 2, 2, 2, 2)),
        ("bn_relu_maxpool2_fwd (3 launches)", 4 * fp + fp // 4 + n // 4, lambda: L.aeth_bn_relu_maxpool2_fwd_f32(
            x.ptr, gamma.ptr, beta.ptr, rm.ptr, rv.ptr, sm.ptr, si.ptr, y.ptr, y2.ptr, pooled.ptr, idx.ptr,
            S, H, W, Ch, f(1e-5), f(0.9), f(0.0))),
        ("maxpool2_relu_bn_bwd (3 launches)", 7 * fp + fp // 4 + n // 4, lambda: L.aeth_maxpool2_relu_bn_bwd_f32(
            dpooled.ptr, idx.ptr, y.ptr, x.ptr, gamma.ptr, sm.ptr, si.ptr, y2.ptr, y3.ptr, y.ptr, dgamma.ptr,
            dbeta.ptr, S, H, W, Ch, f(0.0))),
        ("cast_f32_to_bf16", fp + fp // 2, lambda: L.aeth_cast_f32_to_bf16(x.ptr, y.ptr, i64(n))),
        ("fill_f32", fp, lambda: L.aeth_fill_f32(y.ptr, f(0.0), i64(n))),
        ("memcpy_d2d", 2 * fp, lambda: L.aeth_memcpy_d2d(y.ptr, x.ptr, i64(fp))),
    ]
    out = {}
    for name, nbytes, call in calls:
        ms = _time(lambda: _lib.check(call()), steps, warmup)
        out[name] = {"ms": round(ms, 4), "algorithmic_MB": round(nbytes / 1e6, 1), "TB_per_s": round(nbytes / ms / 1e9, 2)}
    return out


def run(steps, warmup):
    return {"conv_shapes": conv_table(max(20, steps), 2), "bf16_through_the_layer": bf16_layer(max(20, steps), 3),
            "train_step_cnn3": train_step(max(steps, 20), warmup)}


if __name__ == "__main__":
    import json
    if "--bf16-layer" in sys.argv:
        print(json.dumps(bf16_layer(20, 3), indent=1))
    elif "--layers" in sys.argv:
        print(json.dumps(layer_kernels(20, 5), indent=1))
    elif "--train-only" in sys.argv:
        print(json.dumps(train_step(50, 10, eager_only="--eager" in sys.argv), indent=1))
    elif "--shape" in sys.argv:
        # one shape of the list only, e.g. --shape cfg4_1x1_64_to256 (for profiler runs)
        print(json.dumps(conv_table(20, 2, only=sys.argv[sys.argv.index("--shape") + 1]), indent=1))
    else:
        print(json.dumps(run(20, 5), indent=1))
