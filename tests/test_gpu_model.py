"""Whole training step of the three-block CNN (batch 128, 32x32x3 synthetic
images) through the reference's Model API on the GPU, against the float64 CPU
oracle started from the same float32 parameters.

Tolerances.  Scalars and per-tensor parameter gradients: 1e-5*max(1,rms) +
1e-4*|oracle| (the rms scaling is explained in tests/abi.py), applied to the
first step.  Activations' gradients pass through ReLU / max-pool selections,
where a float32 and a float64 evaluation may pick differently for values within
rounding of a tie; those tensors are compared by relative L2 error <= 1e-4 and by
the share of elements outside tolerance <= 1e-4.  The Adam update is checked after
every step by tests/step_checks.py: against the update formula applied to the GPU's
own state (every element, 1e-4*lr) and, after the first step, against the oracle
network's parameter change with the tolerance the gradient bar implies.  The batch
norms' running statistics are compared directly (1e-5 + 1e-3*|oracle|)."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import step_checks as SC

pytestmark = pytest.mark.gpu


def build_model(aether, label_smoothing=0.01, hw=32, in_ch=3):
    m = aether.Model()
    c = in_ch
    size = hw
    for d in (32, 64, 128):
        m.add(aether.Conv_Layer((size, size, c), num_filters=d, filter_size=(3, 3), strides=(1, 1), padding="same"))
        m.add(aether.Batch_Norm())
        m.add(aether.ReLU())
        m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
        c = d
        size //= 2
    m.add(aether.Flatten())
    m.add(aether.Layer_Dense(size * size * 128, 256))
    m.add(aether.Leaky_ReLU(alpha=0.01))
    m.add(aether.Layer_Dense(256, 10))
    m.add(aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(label_smoothing=label_smoothing),
          optimizer=aether.Optimizer_Adam(learning_rate=1e-3),
          accuracy=aether.Accuracy_Categorical())
    m.finalize()
    return m


def host_params(model):
    """Parameter tuples as float32 NumPy arrays; BN running stats that do not exist
    yet (lazy init) are the reference's initial values."""
    out = []
    for layer in model.trainable_layers:
        tup = layer.get_parameters()
        if len(tup) == 4 and tup[0] is None:
            C = layer.prev.filter_weights.shape[3]
            out.append((np.ones(C, np.float32), np.zeros(C, np.float32), np.zeros(C, np.float32),
                        np.ones(C, np.float32)))
        else:
            out.append(tuple(np.asarray(a) for a in tup))
    return out


def rel_l2(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def outside_share(got, want, rtol=1e-4, atol=1e-5):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = max(1.0, float(np.sqrt(np.mean(want * want))))
    return float(np.mean(np.abs(got - want) > atol * scale + rtol * np.abs(want)))


def test_three_block_cnn_training_steps_match_oracle(capsys):
    import aether
    from tests import abi
    np.random.seed(0)
    X = np.random.rand(128, 32, 32, 3).astype(np.float32)
    y = np.random.randint(0, 10, 128)
    model = build_model(aether)
    assert [type(l).__name__ for l in model.trainable_layers] == \
        ["Conv_Layer", "Batch_Norm"] * 3 + ["Layer_Dense", "Layer_Dense"]
    assert model.softmax_classifier_output is not None
    params = host_params(model)
    n_params = sum(int(np.prod(a.shape)) for tup in params for a in tup[:2])
    assert n_params == 620810
    net = O.OracleCNN(params, label_smoothing=0.01, lr=1e-3, dtype=np.float64)

    model.loss.new_pass()
    model.accuracy.new_pass()
    for step in range(3):
        before = SC.snapshot(model)
        ref = net.step(X, y)
        loss, data_loss, reg_loss, acc = model.train_step(X, y)
        assert reg_loss == 0
        assert abs(loss - ref["loss"]) <= 1e-5 + 1e-4 * abs(ref["loss"]), (step, loss, ref["loss"])
        assert abs(acc - ref["acc"]) <= 1.0 / 128 + 1e-9
        probs = model.layers[-1].output.get()
        assert rel_l2(probs, ref["probs"]) <= (1e-4 if step == 0 else 2e-3)
        if step == 0:
            abi.close(probs, ref["probs"])
            for i, layer in enumerate(model.trainable_layers):
                gw, gb = ref["grads"][i]
                name = "%d:%s" % (i, type(layer).__name__)
                assert rel_l2(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 2e-4, name
                assert outside_share(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 1e-3, name
                if np.linalg.norm(gb) > 1e-12:          # conv biases feed a batch norm: gradient is 0
                    assert rel_l2(layer.dbiases.get(), gb.reshape(layer.dbiases.shape)) <= 2e-4, name
                else:
                    assert np.abs(layer.dbiases.get()).max() <= 1e-5, name
            convs = [l for l in model.layers if isinstance(l, aether.Conv_Layer)]
            for blk, conv in enumerate(convs):
                want = ref["dinputs"]["conv%d" % blk]
                assert conv.dinputs.shape == want.shape
                assert rel_l2(conv.dinputs.get(), want) <= 2e-4, blk
                assert outside_share(conv.dinputs.get(), want) <= 1e-3, blk
        SC.check_update_from_own_state(model, before, 1e-3, step)
        if step == 0:
            SC.check_update_against_oracle(model, before, net.p, ref["grads"], 1e-3)
        for i, layer in enumerate(model.trainable_layers):
            got = [np.asarray(a) for a in layer.get_parameters()]
            for j, want in enumerate(net.p[i]):
                if j >= 2:                                  # BN running statistics
                    g = got[j].reshape(want.shape)
                    assert np.all(np.abs(g - want) <= 1e-5 + 1e-3 * np.abs(want)), (step, i, j)
    assert model.optimizer.iterations == 3
    assert model.loss.accumulated_count == 3 * 128

    # evaluation path (running statistics, no smoothing) and predict()
    probs_eval, _ = net.forward(X, training=False)
    pred = model.predict(X, batch_size=50)                  # ragged last batch
    assert pred.shape == (128, 10)
    assert rel_l2(pred, probs_eval) <= 5e-3
    model.evaluate(X, y, batch_size=64)
    out = capsys.readouterr().out
    assert "Valdiation, acc:" in out
    want_loss = float(np.mean(O.cce_forward(probs_eval, y, 0.01, training=False)))
    assert abs(float(model.loss.calculate_accumulated()) - want_loss) <= 5e-3 * max(1.0, want_loss)


def test_train_prints_reference_format_and_parameters_round_trip(tmp_path, capsys):
    import aether
    np.random.seed(3)
    X = np.random.rand(48, 16, 16, 3).astype(np.float32)
    y = np.random.randint(0, 10, 48)
    model = build_model(aether, hw=16)
    model.train(X, y, epochs=2, batch_size=20, print_every=2, validation_data=(X, y))
    out = capsys.readouterr().out.splitlines()
    assert out[0] == "Training" and out[1] == " epoch: 1"
    step_lines = [l for l in out if l.startswith("epoch: ")]
    assert len(step_lines) == 4                              # steps 0 and 2 of each epoch
    assert step_lines[0].startswith("epoch: 1, acc: 0.") and ", loss: " in step_lines[0]
    assert "(data_loss: " in step_lines[0] and "reg_loss: 0.000, lr:: 0.001" in step_lines[0]
    assert any(l.startswith(" training, acc: ") for l in out)
    assert any(l.startswith("Valdiation, acc: ") for l in out)

    path = str(tmp_path / "params.pkl")
    model.save_parameters(path)
    before = model.predict(X)
    np.random.seed(4)
    other = build_model(aether, hw=16)
    other.forward(X[:4], training=False)                     # lazily creates the BN tensors
    other.load_parameters(path)
    assert other.layers[0].weights is other.layers[0].filter_weights
    after = other.predict(X)
    assert np.array_equal(before, after)
    # the same through a file written the way the reference's CuPy model writes its checkpoints
    path2 = str(tmp_path / "params_cupy.pkl")
    model.save_parameters(path2, cupy_arrays=True)
    assert b"cupy._core.core" in open(path2, "rb").read()
    # with the reference's dtypes: float64 dense parameters (CNN_classes_cupy.py:320-322), float32 everything else
    import io
    from aether.model import _ArrayOnlyUnpickler
    stored = _ArrayOnlyUnpickler(io.BytesIO(open(path2, "rb").read())).load()
    kinds = [type(l).__name__ for l in model.trainable_layers]
    for kind, tup in zip(kinds, stored):
        assert all(a.dtype == (np.float64 if kind == "Layer_Dense" else np.float32) for a in tup), kind
    np.random.seed(5)
    third = build_model(aether, hw=16)
    third.forward(X[:4], training=False)
    third.load_parameters(path2)
    assert np.array_equal(before, third.predict(X))
    with pytest.raises(Exception):
        bad = tmp_path / "bad.pkl"
        import pickle
        bad.write_bytes(pickle.dumps([(__import__("os").getcwd,)]))
        other.load_parameters(str(bad))


def test_load_parameters_accepts_cupy_wrapped_float64_checkpoints(tmp_path):
    """The reference's CuPy checkpoints pickle every array as
    cupy._core.core.array(ndarray), dense weights in float64 and BN running stats
    with shape (1,1,1,C).  A file with that structure (written here, synthetic
    values) loads without CuPy."""
    import pickle
    import aether

    class _Wrapped:                                           # pickles as cupy._core.core.array(ndarray)
        def __init__(self, a):
            self.a = a

        def __reduce__(self):
            return (_FakeCupyArray, (self.a,))

    class _FakeCupyArray:
        pass
    _FakeCupyArray.__module__ = "cupy._core.core"
    _FakeCupyArray.__qualname__ = _FakeCupyArray.__name__ = "array"

    import sys
    import types
    mods = {}
    for name in ("cupy", "cupy._core", "cupy._core.core"):
        mods[name] = types.ModuleType(name)
    mods["cupy._core.core"].array = _FakeCupyArray
    sys.modules.update(mods)
    try:
        r = np.random.RandomState(5)
        params = [
            (r.randn(3, 3, 1, 32).astype(np.float32), r.randn(32).astype(np.float32)),
            (r.rand(32).astype(np.float32) + 0.5, r.randn(32).astype(np.float32),
             r.randn(1, 1, 1, 32).astype(np.float32), r.rand(1, 1, 1, 32).astype(np.float32) + 0.5),
            (r.randn(6272, 10) * 0.01, r.randn(1, 10)),       # float64 dense
        ]
        blob = pickle.dumps([tuple(_Wrapped(a) for a in tup) for tup in params], protocol=4)
    finally:
        for name in mods:
            sys.modules.pop(name, None)
    assert b"cupy._core.core" in blob
    path = tmp_path / "cupy_style"
    path.write_bytes(blob)

    m = aether.Model()
    m.add(aether.Conv_Layer((28, 28, 1), num_filters=32))
    m.add(aether.Batch_Norm())
    m.add(aether.ReLU())
    m.add(aether.Pooling())
    m.add(aether.Flatten())
    m.add(aether.Layer_Dense(6272, 10))
    m.add(aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(), optimizer=aether.Optimizer_Adam(),
          accuracy=aether.Accuracy_Categorical())
    m.finalize()
    m.load_parameters(str(path))
    x = r.rand(5, 28, 28, 1).astype(np.float32)
    got = m.predict(x)
    W, b = params[0]
    a = O.conv_fprop(x, W, b, (1, 1), "same", dtype=np.float64)
    g, be, rm, rv = (p.astype(np.float64) for p in params[1])
    a = O.relu_forward(O.bn_forward_infer(a, g, be, rm, rv, 1e-5))
    a, _ = O.maxpool_forward(a, dtype=np.float64)
    want = O.softmax(O.dense_forward(a.reshape(5, -1), params[2][0], params[2][1], dtype=np.float64))
    from tests import abi
    abi.close(got, want, rtol=1e-3)


@pytest.mark.parametrize("switches", [{}, {"gather_border": 1}], ids=["as the shapes decide", "fprop and dgrad cut along their borders"])
def test_recorded_steps_equal_eager_steps(switches, tune):
    """Model.record_steps: a step replayed from a HIP graph must give what the same
    step gives when every kernel is launched from Python.  Same kernels in the same
    order, so the comparison is exact.  The replays are interleaved with eager work
    of the same model (an evaluation, a step of another batch shape, a
    synchronisation), every replay is checked, and learning-rate decay is on so that
    the step state kept on the device matters.  Second run: the convolutions' forward
    and input-gradient products cut into their border parts, nine problems per launch
    (what large layers get), so that these launches are recorded and replayed too."""
    import aether
    from aether import _lib
    tune(**switches)

    def make():
        np.random.seed(3)
        m = build_model(aether, hw=16)
        m.optimizer.decay = 1e-2
        m.loss.new_pass()
        m.accuracy.new_pass()
        return m

    rng = np.random.RandomState(5)
    Xs = [rng.rand(32, 16, 16, 3).astype(np.float32) for _ in range(3)]
    ys = [rng.randint(0, 10, 32) for _ in range(3)]
    Xodd, yodd = rng.rand(16, 16, 16, 3).astype(np.float32), rng.randint(0, 10, 16)
    eager, rec = make(), make()
    rec.record_steps(True)
    for step in range(9):
        X, y = Xs[step % 3], ys[step % 3]
        a = eager.train_step(X, y)
        b = rec.train_step(X, y)
        assert a == b, "step %d: eager %r, recorded %r" % (step, a, b)
        assert eager.optimizer.iterations == rec.optimizer.iterations
        assert eager.optimizer.current_learning_rate == rec.optimizer.current_learning_rate
        for la, lb in zip(eager.trainable_layers, rec.trainable_layers):
            assert np.array_equal(np.asarray(la.weights), np.asarray(lb.weights)), "weights differ after step %d" % step
            assert np.array_equal(np.asarray(la.dweights), np.asarray(lb.dweights)), "layer.dweights is stale"
        if step == 4:
            for m in (eager, rec):
                m.evaluate(Xs[0], ys[0], batch_size=16)
            _lib.sync()
        if step == 6:
            assert eager.train_step(Xodd, yodd) == rec.train_step(Xodd, yodd)      # another shape: runs eagerly
        if step == 7:
            # parameters set anew live in new buffers: the recording made with the old ones must not be replayed
            for m in (eager, rec):
                host = [tuple(np.array(np.asarray(t)) for t in ps) for ps in m.get_parameters()]
                m.set_parameters(host)
    assert len([r for r in rec._recordings.values() if r.get("graph")]) == 1
    rec.record_steps(False)
    assert eager.train_step(Xs[0], ys[0]) == rec.train_step(Xs[0], ys[0])


def test_classifier_head_in_one_launch_equals_the_three_launches(monkeypatch):
    """A training step queues softmax, loss + predictions and the gradient of the logits as one launch
    (AETHER_FUSE_HEAD=0: the three launches of the layers).  Same operations in the same order: the
    steps must agree exactly, eager and recorded, and the layer attributes must be those of the step."""
    import aether

    def run(fuse, record):
        monkeypatch.setenv("AETHER_FUSE_HEAD", fuse)
        np.random.seed(3)
        m = build_model(aether, label_smoothing=0.05, hw=16)
        m.loss.new_pass()
        m.accuracy.new_pass()
        m.record_steps(record)
        rng = np.random.RandomState(5)
        out = []
        for step in range(5):
            X, y = rng.rand(32, 16, 16, 3).astype(np.float32), rng.randint(0, 10, 32)
            out.append(m.train_step(X, y))
        return out, np.asarray(m.layers[-1].output), np.asarray(m.layers[-1].dinputs), \
            [np.asarray(l.weights) for l in m.trainable_layers]

    ref = run("0", False)
    for fuse, record in (("1", False), ("1", True)):
        got = run(fuse, record)
        assert got[0] == ref[0]
        assert np.array_equal(got[1], ref[1]) and np.array_equal(got[2], ref[2])
        for a, b in zip(got[3], ref[3]):
            assert np.array_equal(a, b)


def test_recorded_steps_survive_a_workspace_that_grows():
    """A recorded step has the address of the library's scratch workspace in its kernel
    arguments.  Eager work that needs a larger workspace after the recording was made
    (here a wgrad whose split partials take tens of MB) replaces the workspace; the old
    one must stay valid for the replays that follow."""
    import aether
    from tests import abi

    def make():
        np.random.seed(4)
        m = build_model(aether, hw=16)
        m.loss.new_pass()
        m.accuracy.new_pass()
        return m

    rng = np.random.RandomState(6)
    X, y = rng.rand(32, 16, 16, 3).astype(np.float32), rng.randint(0, 10, 32)
    eager, rec = make(), make()
    rec.record_steps(True)
    for step in range(3):                                    # normal, recorded, replayed
        assert eager.train_step(X, y) == rec.train_step(X, y)
    assert any(r.get("graph") for r in rec._recordings.values())
    xb = rng.randn(64, 56, 56, 64).astype(np.float32)
    dyb = rng.randn(64, 56, 56, 64).astype(np.float32)
    dw1, _ = abi.wgrad(xb, dyb, (3, 3, 64, 64), (1, 1), "same")      # grows the workspace
    for step in range(3):
        a, b = eager.train_step(X, y), rec.train_step(X, y)
        assert a == b, "replay %d after the workspace grew: eager %r, recorded %r" % (step, a, b)
        for la, lb in zip(eager.trainable_layers, rec.trainable_layers):
            assert np.array_equal(np.asarray(la.weights), np.asarray(lb.weights))
        dw2, _ = abi.wgrad(xb, dyb, (3, 3, 64, 64), (1, 1), "same")  # eager work in the new workspace between replays
        assert np.array_equal(dw1, dw2)
    rec.record_steps(False)


def test_recording_refuses_calls_that_wait_for_the_device():
    import ctypes as C
    import aether
    from aether import _lib
    lib = _lib.lib()
    t = aether.DeviceTensor.zeros(8)
    _lib.sync()
    _lib.check(lib.aeth_graph_begin())
    try:
        assert lib.aeth_sync() == _lib.AETH_E_STATE
        host = np.zeros(8, np.float32)
        assert lib.aeth_memcpy_d2h(host.ctypes.data, t.ptr, 32) == _lib.AETH_E_STATE
        assert lib.aeth_graph_begin() == _lib.AETH_E_STATE
        ev = _lib.Event()
        assert lib.aeth_event_record(ev._h) == _lib.AETH_E_STATE
        _lib.check(lib.aeth_fill_f32(t.ptr, 2.0, 8))
    finally:
        g = C.c_void_p()
        rc = lib.aeth_graph_end(C.byref(g))
    _lib.check(rc)
    assert np.all(t.get() == 0)                     # recorded, not run
    for _ in range(3):
        _lib.check(lib.aeth_fill_f32(t.ptr, 1.0, 8))
        _lib.check(lib.aeth_graph_launch(g))
        assert np.all(t.get() == 2)
    _lib.check(lib.aeth_graph_destroy(g))
    assert lib.aeth_graph_end(C.byref(g)) == _lib.AETH_E_STATE


def test_backward_debug_prints_the_reference_lines(capsys):
    """Model.backward_debug (CNN_model_cupy.py:195-229), as the reference's scripts call it on one sample
    (CNN/architectures/CNN_test2.py:75): every layer's output shape, then every layer's gradient shapes walking back."""
    import aether
    np.random.seed(11)
    X = np.random.rand(1, 16, 16, 3).astype(np.float32)
    y = np.random.randint(0, 10, 1)
    model = build_model(aether, hw=16)
    before = [np.asarray(p) for layer in model.trainable_layers if type(layer).__name__ != "Batch_Norm"
              for p in layer.get_parameters()]
    model.backward_debug(X, y)
    out = capsys.readouterr().out.splitlines()
    assert out[0] == "Forward pass:"
    assert out[1] == "Layer 0 (Conv_Layer) output: (1, 16, 16, 32)"
    assert out[len(model.layers)] == "Layer %d (SoftMax) output: (1, 10)" % (len(model.layers) - 1)
    i = out.index("Backward pass:")
    assert out[i - 1] == ""
    assert out[i + 1] == "Layer -2 (Layer_Dense) dinputs: (1, 256)"
    assert out[i + 2] == "             dweights: (256, 10)"
    assert out[i + 3] == "             dbiases: (1, 10)"
    assert out[-3] == "Layer -%d (Conv_Layer) dinputs: (1, 16, 16, 3)" % len(model.layers)
    assert out[-2] == "             dweights: (3, 3, 3, 32)" and out[-1] == "             dbiases: (32,)"
    after = [np.asarray(p) for layer in model.trainable_layers if type(layer).__name__ != "Batch_Norm"
             for p in layer.get_parameters()]
    assert all(np.array_equal(a, b) for a, b in zip(before, after))
