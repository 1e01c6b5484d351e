"""Whole training steps of the reference's shipped CIFAR recipe
(CNN/architectures/CNN_cifar1.py:19-55) on the GPU against the float64 oracle:
Conv(32)-BN-ReLU-Pool, Conv(64)-BN-ReLU-SpatialDropout(0.075)-Pool,
Conv(128)-BN-ReLU-SpatialDropout(0.1)-Pool, Flatten, Dense(2048,256; L2 2e-5 on weights
and biases)-LeakyReLU(0.01)-Dropout(0.075), Dense(256,10), softmax cross-entropy with
label smoothing 0.01, Adam(lr 1e-3, decay 5e-5), batch 128.

Dropout masks are drawn on the host with the reference's shapes ((1,1,1,C)/keep and
elementwise/keep) and handed to both sides (`fixed_mask` on the layers, `masks=` on the
oracle), a fresh set every step.  Tolerances as in tests/test_gpu_model.py."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import step_checks as SC
from tests.test_gpu_model import host_params, outside_share, rel_l2

pytestmark = pytest.mark.gpu


def cifar1_model(aether):
    m = aether.Model()
    m.add(aether.Conv_Layer(input_shape=(32, 32, 3), num_filters=32, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Batch_Norm(epsilon=1e-5, momentum=0.9))
    m.add(aether.ReLU())
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Conv_Layer(input_shape=(16, 16, 32), num_filters=64, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Batch_Norm(epsilon=1e-5, momentum=0.9))
    m.add(aether.ReLU())
    m.add(aether.Layer_Dropout_Spatial(rate=0.075))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Conv_Layer(input_shape=(8, 8, 64), num_filters=128, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Batch_Norm(epsilon=1e-5, momentum=0.9))
    m.add(aether.ReLU())
    m.add(aether.Layer_Dropout_Spatial(rate=0.1))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Flatten())
    m.add(aether.Layer_Dense(4 * 4 * 128, n_neurons=256, weight_regularizer_l2=2e-5, bias_regularizer_l2=2e-5))
    m.add(aether.Leaky_ReLU(alpha=0.01))
    m.add(aether.Layer_Dropout(rate=0.075))
    m.add(aether.Layer_Dense(256, 10))
    m.add(aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(label_smoothing=0.01),
          optimizer=aether.Optimizer_Adam(learning_rate=0.001, decay=5e-5),
          accuracy=aether.Accuracy_Categorical())
    m.finalize()
    return m


def draw_masks(rng, S):
    """Bernoulli(keep)/keep with the reference's shapes (CNN_classes_cupy.py:375-376, :397-398)."""
    return {"spatial1": (rng.binomial(1, 1 - 0.075, size=(1, 1, 1, 64)) / (1 - 0.075)).astype(np.float32),
            "spatial2": (rng.binomial(1, 1 - 0.1, size=(1, 1, 1, 128)) / (1 - 0.1)).astype(np.float32),
            "dense": (rng.binomial(1, 1 - 0.075, size=(S, 256)) / (1 - 0.075)).astype(np.float32)}


@pytest.mark.parametrize("recorded", [False, True], ids=["eager", "recorded"])
def test_cifar1_recipe_steps_match_oracle(recorded):
    """`recorded`: the same steps through Model.record_steps(True): step 0 runs eagerly, step 1 is recorded as a HIP
    graph and launched, steps 2 and 3 replay it with that step's masks copied into the buffers the graph reads."""
    import aether
    from tests import abi
    np.random.seed(0)
    S = 128
    X = np.random.rand(S, 32, 32, 3).astype(np.float32)
    y = np.random.randint(0, 10, S)
    model = cifar1_model(aether)
    # Dense-1's fresh weights are ~1e-4 (the reference's 0.01 factor): its penalty would be
    # 2e-5 * 0.03 and invisible next to the data loss.  Scale them so that the L2 terms matter.
    d1 = [l for l in model.layers if isinstance(l, aether.Layer_Dense)][0]
    d1.set_parameters(np.asarray(d1.weights) * 200, np.full((1, 256), 0.5, np.float32))
    spatial = [l for l in model.layers if isinstance(l, aether.Layer_Dropout_Spatial)]
    dense_drop = [l for l in model.layers if isinstance(l, aether.Layer_Dropout)][0]
    params = host_params(model)
    net = O.OracleCNN(params, label_smoothing=0.01, lr=1e-3, decay=5e-5, dtype=np.float64, dense1_l2=(2e-5, 2e-5))

    if recorded:
        model.record_steps(True)
        assert model.recording_active is True
    model.loss.new_pass()
    model.accuracy.new_pass()
    rng = np.random.RandomState(9)
    for step in range(4):
        masks = draw_masks(rng, S)
        spatial[0].fixed_mask, spatial[1].fixed_mask, dense_drop.fixed_mask = \
            masks["spatial1"], masks["spatial2"], masks["dense"]
        before = SC.snapshot(model)
        ref = net.step(X, y, masks=masks)
        loss, data_loss, reg_loss, acc = model.train_step(X, y)
        assert ref["reg_loss"] > 1e-3                       # the penalty is visible at the printed precision
        assert abs(data_loss - ref["loss"]) <= 1e-5 + 1e-4 * abs(ref["loss"]), (step, data_loss, ref["loss"])
        assert abs(reg_loss - ref["reg_loss"]) <= 1e-6 + 1e-4 * ref["reg_loss"], (step, reg_loss, ref["reg_loss"])
        assert abs(loss - (ref["loss"] + ref["reg_loss"])) <= 2e-5 + 1e-4 * abs(loss)
        assert abs(acc - ref["acc"]) <= 1.0 / S + 1e-9
        assert model.optimizer.current_learning_rate == pytest.approx(1e-3 / (1 + 5e-5 * step), rel=1e-12)
        assert model.optimizer.current_learning_rate == pytest.approx(ref["lr"], rel=1e-12)
        # the masks the layers used are the ones handed in, in the reference's shapes
        assert np.array_equal(spatial[0].channel_mask.get(), masks["spatial1"])
        assert np.array_equal(spatial[1].channel_mask.get(), masks["spatial2"])
        assert np.array_equal(dense_drop.binary_mask.get(), masks["dense"])
        probs = model.layers[-1].output.get()
        assert rel_l2(probs, ref["probs"]) <= (1e-4 if step == 0 else 2e-3)
        if step == 0:
            abi.close(probs, ref["probs"])
            for i, layer in enumerate(model.trainable_layers):
                gw, gb = ref["grads"][i]
                name = "%d:%s" % (i, type(layer).__name__)
                assert rel_l2(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 2e-4, name
                assert outside_share(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 1e-3, name
                if np.linalg.norm(gb) > 1e-12:
                    assert rel_l2(layer.dbiases.get(), gb.reshape(layer.dbiases.shape)) <= 2e-4, name
                else:
                    assert np.abs(layer.dbiases.get()).max() <= 1e-5, name
            # Dense-1's gradient carries 2*lambda*W: without it the comparison above fails
            gw = ref["grads"][6][0]
            assert rel_l2(gw - 2 * 2e-5 * params[6][0].astype(np.float64), gw) > 1e-3
            convs = [l for l in model.layers if isinstance(l, aether.Conv_Layer)]
            for blk, conv in enumerate(convs):
                want = ref["dinputs"]["conv%d" % blk]
                assert rel_l2(conv.dinputs.get(), want) <= 2e-4, blk
                assert outside_share(conv.dinputs.get(), want) <= 1e-3, blk
        # Adam with the decayed learning rate of this step (tests/step_checks.py)
        SC.check_update_from_own_state(model, before, ref["lr"], step)
        if step == 0:
            SC.check_update_against_oracle(model, before, net.p, ref["grads"], ref["lr"])
        for i, layer in enumerate(model.trainable_layers):
            got = [np.asarray(a) for a in layer.get_parameters()]
            for j, want in enumerate(net.p[i]):
                if j >= 2 and step < 3:                     # BN running statistics (float32 and float64 parameters drift apart from step to step)
                    g = got[j].reshape(want.shape)
                    assert np.all(np.abs(g - want) <= 1e-5 + 1e-3 * np.abs(want)), (step, i, j)
    assert model.optimizer.iterations == 4
    assert len([r for r in getattr(model, "_recordings", {}).values() if r.get("graph")]) == (1 if recorded else 0)

    # evaluation: dropout layers pass their input through, no smoothing
    probs_eval, _ = net.forward(X, training=False)
    pred = model.predict(X, batch_size=64)
    assert rel_l2(pred, probs_eval) <= 5e-3


def test_cifar1_recipe_recorded_steps_draw_the_same_masks_as_eager_steps():
    """Without `fixed_mask` the layers draw their masks from the legacy global RNG, as the reference does.  A
    recorded step draws them on the host in the layers' order before the replay: the same random stream as the
    eager step, so losses and parameters agree bit for bit, replay after replay, and the masks differ from
    step to step."""
    import aether
    rng = np.random.RandomState(21)
    Xs = [rng.rand(128, 32, 32, 3).astype(np.float32) for _ in range(2)]
    ys = [rng.randint(0, 10, 128) for _ in range(2)]

    def run(record):
        np.random.seed(13)
        model = cifar1_model(aether)
        d1 = [l for l in model.layers if isinstance(l, aether.Layer_Dense)][0]
        d1.set_parameters(np.asarray(d1.weights) * 200, np.full((1, 256), 0.5, np.float32))
        model.record_steps(record)
        model.loss.new_pass()
        model.accuracy.new_pass()
        np.random.seed(14)
        out, masks = [], []
        drop = [l for l in model.layers if isinstance(l, aether.Layer_Dropout)][0]
        for step in range(6):
            out.append(model.train_step(Xs[step % 2], ys[step % 2]))
            masks.append(drop.binary_mask.get())
        params = [np.asarray(p) for layer in model.trainable_layers for p in layer.get_parameters()]
        return out, masks, params, model

    eager, masks_e, params_e, _ = run(False)
    rec, masks_r, params_r, model = run(True)
    assert model.recording_active
    assert len([r for r in model._recordings.values() if r.get("graph")]) == 1
    assert eager == rec, (eager, rec)
    assert all(np.array_equal(a, b) for a, b in zip(masks_e, masks_r))
    assert not np.array_equal(masks_r[3], masks_r[4])        # a fresh draw every replay
    assert 0.85 < float((masks_r[4] > 0).mean()) < 0.98      # keep probability 0.925
    assert all(np.array_equal(a, b) for a, b in zip(params_e, params_r))


def test_train_reads_steps_one_step_late_and_prints_the_same_lines(capsys):
    """Model.train queues step k + 1 before it reads step k's loss and predictions, with steps launched kernel by kernel
    and with replayed ones.  The printed lines (every second step and the last of an epoch, the summary, the validation
    line), the accumulated sums and the parameters are those of a loop that reads every step at once; the last batch of
    an epoch is ragged (another shape: with recorded steps it runs normally in the first epoch, is recorded in the second
    and replayed in the third)."""
    import aether
    rng = np.random.RandomState(31)
    X = rng.rand(150, 32, 32, 3).astype(np.float32)
    y = rng.randint(0, 10, 150)
    outs, params = [], []
    for mode in ("at once", "late", "recorded"):
        np.random.seed(17)
        model = cifar1_model(aether)
        model.record_steps(mode == "recorded")
        if mode == "at once":                                # every step's scalars read before the next step is queued
            plain = model._eager_step
            model._eager_step = lambda bx, by, later=False: plain(bx, by)
        np.random.seed(18)                                   # the dropout masks' random stream
        model.train(X, y, epochs=3, batch_size=32, print_every=2, validation_data=(X[:40], y[:40]))
        outs.append(capsys.readouterr().out)
        params.append([np.asarray(p) for layer in model.trainable_layers for p in layer.get_parameters()])
        if mode == "recorded":
            assert len([r for r in model._recordings.values() if r.get("graph")]) == 2
    assert outs[0] == outs[1] == outs[2]
    assert outs[0].count("epoch: ") == 3 + 3 * 3             # the epoch headers and steps 0, 2, 4 of each
    assert all(np.array_equal(a, b) and np.array_equal(a, c) for a, b, c in zip(*params))


def test_two_part_copies_to_the_host():
    """aeth_d2h_begin / aeth_d2h_end: the bytes are those of the moment the copy was queued, whatever is queued
    behind it; at most 8 may be pending; a ticket is ended once."""
    import ctypes as C
    from aether import _lib
    from aether.tensor import DeviceTensor
    lib = _lib.lib()
    t = DeviceTensor.from_numpy(np.arange(1000, dtype=np.float32))
    later = t.get_later()
    t.fill(7.0)                                              # queued behind the copy
    assert np.array_equal(later(), np.arange(1000, dtype=np.float32))
    assert np.all(t.get() == 7.0)
    pending = [DeviceTensor.from_numpy(np.full(16, k, np.float32)).get_later() for k in range(8)]
    ticket = C.c_int(-1)
    assert lib.aeth_d2h_begin(t.ptr, 64, C.byref(ticket)) == _lib.AETH_E_STATE        # a ninth
    big = DeviceTensor.zeros(1 << 20)
    big.set(np.ones(1 << 20, np.float32))                    # a 4 MB upload passes over the held slots
    assert [int(p()[0]) for p in pending] == list(range(8))
    assert lib.aeth_d2h_end(0, None, 0) == _lib.AETH_E_INVALID                          # nothing pending there
    assert np.all(big.get_later()() == 1.0) if big.nbytes <= 256 * 1024 else np.all(big.get() == 1.0)
    assert lib.aeth_d2h_begin(t.ptr, 1 << 20, C.byref(ticket)) == _lib.AETH_E_INVALID   # more than a slot holds
