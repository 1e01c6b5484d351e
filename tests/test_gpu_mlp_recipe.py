"""Whole training steps of the reference's dense-only recipe (CNN/architectures/CNN_cifar2.py:13-34,
the same network as CNN_test_cupy.py:33-50) on the GPU against the float64 oracle: flattened
32x32x3 images, Dense(3072,256)-ReLU-Dense(256,256)-ReLU-Dense(256,256)-ReLU, each with L2 5e-5 on
weights and biases, Dense(256,32)-ReLU-Dense(32,10)-SoftMax, Loss_CategoricalCrossEntropy(),
Adam(decay 1e-4), batch 128.

The `Layer_Dense` half of the path as a model of its own: products with 3072, 256 and 32 input
columns and 256, 32 and 10 output columns, the regulariser sum over three layers, and
`Model.train` itself with the recipe's arguments."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import step_checks as SC
from tests.test_gpu_model import host_params, outside_share, rel_l2

pytestmark = pytest.mark.gpu

L2 = 5e-5
LR, DECAY = 1e-3, 1e-4
WIDTHS = [(3072, 256, L2), (256, 256, L2), (256, 256, L2), (256, 32, 0.0), (32, 10, 0.0)]


def mlp_model(aether):
    m = aether.Model()
    for i, (n_in, n_out, l2) in enumerate(WIDTHS):
        if l2:
            m.add(aether.Layer_Dense(n_in, n_out, weight_regularizer_l2=l2, bias_regularizer_l2=l2))
        else:
            m.add(aether.Layer_Dense(n_in, n_out))
        m.add(aether.ReLU() if i + 1 < len(WIDTHS) else aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(), optimizer=aether.Optimizer_Adam(decay=DECAY),
          accuracy=aether.Accuracy_Categorical())
    m.finalize()
    return m


class OracleMlp:
    def __init__(self, params):
        self.p = [[np.array(a, dtype=np.float64) for a in tup] for tup in params]
        self.m = [[np.zeros_like(a) for a in tup] for tup in self.p]
        self.v = [[np.zeros_like(a) for a in tup] for tup in self.p]
        self.iterations = 0

    def forward(self, X):
        a = np.asarray(X, dtype=np.float64)
        ins, pre = [], []
        for i, (W, b) in enumerate(self.p):
            ins.append(a)
            a = O.dense_forward(a, W, b, dtype=np.float64)
            pre.append(a)
            if i + 1 < len(self.p):
                a = O.relu_forward(a)
        return O.softmax(a), ins, pre

    def step(self, X, y):
        probs, ins, pre = self.forward(X)
        loss = float(np.mean(O.cce_forward(probs, y, 0.0, training=True)))
        reg = sum(O.regularization_loss(W, b, wl2=l2, bl2=l2) for (W, b), (_, _, l2) in zip(self.p, WIDTHS))
        acc = float(np.mean(np.argmax(probs, axis=1) == y))
        grads = [None] * len(self.p)
        d = O.softmax_cce_backward(probs, y, 0.0)
        for i in range(len(self.p) - 1, -1, -1):
            if i + 1 < len(self.p):
                d = O.relu_backward(pre[i], d)
            l2 = WIDTHS[i][2]
            dw, db, d = O.dense_backward(ins[i], self.p[i][0], self.p[i][1], d, wl2=l2, bl2=l2, dtype=np.float64)
            grads[i] = (dw, db)
        lr = LR * (1.0 / (1.0 + DECAY * self.iterations))
        for i, tup in enumerate(self.p):
            for j in range(2):
                g = np.asarray(grads[i][j]).reshape(tup[j].shape)
                self.p[i][j], self.m[i][j], self.v[i][j] = O.adam_update(tup[j], g, self.m[i][j], self.v[i][j], lr,
                                                                         self.iterations)
        self.iterations += 1
        return {"loss": loss, "reg_loss": reg, "acc": acc, "probs": probs, "grads": grads, "lr": lr}


def _scaled(model, aether):
    """Fresh dense weights are ~1e-4 (the reference's 0.01 factor): scale them so that the logits, the gradients of the
    early layers and the L2 terms are far from rounding noise."""
    for layer, factor in zip([l for l in model.layers if isinstance(l, aether.Layer_Dense)], (60, 100, 100, 100, 100)):
        layer.set_parameters(np.asarray(layer.weights) * factor, np.full(np.asarray(layer.biases).shape, 0.1, np.float32))


def test_mlp_recipe_steps_match_oracle():
    import aether
    from tests import abi
    np.random.seed(5)
    S = 128
    X = np.random.rand(S, 3072).astype(np.float32)
    y = np.random.randint(0, 10, S)
    model = mlp_model(aether)
    _scaled(model, aether)
    params = host_params(model)
    net = OracleMlp(params)
    model.loss.new_pass()
    model.accuracy.new_pass()
    for step in range(3):
        before = SC.snapshot(model)
        ref = net.step(X, y)
        loss, data_loss, reg_loss, acc = model.train_step(X, y)
        assert ref["reg_loss"] > 1e-3
        assert abs(data_loss - ref["loss"]) <= 1e-5 + 1e-4 * abs(ref["loss"]), (step, data_loss, ref["loss"])
        assert abs(reg_loss - ref["reg_loss"]) <= 1e-6 + 1e-4 * ref["reg_loss"], (step, reg_loss, ref["reg_loss"])
        assert abs(acc - ref["acc"]) <= 1.0 / S + 1e-9
        assert model.optimizer.current_learning_rate == pytest.approx(ref["lr"], rel=1e-12)
        probs = model.layers[-1].output.get()
        assert rel_l2(probs, ref["probs"]) <= (1e-4 if step == 0 else 2e-3)
        if step == 0:
            abi.close(probs, ref["probs"])
            for i, layer in enumerate(model.trainable_layers):
                gw, gb = ref["grads"][i]
                assert rel_l2(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 2e-4, i
                assert outside_share(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 1e-3, i
                assert rel_l2(layer.dbiases.get(), gb.reshape(layer.dbiases.shape)) <= 2e-4, i
        SC.check_update_from_own_state(model, before, ref["lr"], step)
        if step == 0:
            SC.check_update_against_oracle(model, before, net.p, ref["grads"], ref["lr"])
    probs_eval, _, _ = net.forward(X)
    assert rel_l2(model.predict(X, batch_size=50), probs_eval) <= 5e-3


def test_mlp_recipe_train_loop_prints_the_reference_lines(capsys):
    """Model.train on the recipe (CNN_cifar2.py:37-38 with fewer rows): the reference's progress lines
    (CNN_model_cupy.py:128-151), and the same parameters as the same steps taken one by one."""
    import aether
    np.random.seed(6)
    X = np.random.rand(300, 3072).astype(np.float32)
    y = np.random.randint(0, 10, 300)
    np.random.seed(7)
    a = mlp_model(aether)
    np.random.seed(7)
    b = mlp_model(aether)
    _scaled(a, aether)
    _scaled(b, aether)
    a.train(X, y, validation_data=(X[:100], y[:100]), epochs=2, batch_size=128, print_every=100)
    out = capsys.readouterr().out
    assert out.count(" epoch: ") == 2 and "Training" in out and "Valdiation, acc:" in out             # (the reference's spelling, CNN_model_cupy.py:265)
    assert out.count("reg_loss:") >= 5                      # steps 0 and 2 of both epochs and the summary
    b.accuracy.init(y)
    for epoch in range(2):
        b.loss.new_pass()
        b.accuracy.new_pass()
        for lo in range(0, 300, 128):
            b.train_step(X[lo:lo + 128], y[lo:lo + 128])
    for la, lb in zip(a.trainable_layers, b.trainable_layers):
        for pa, pb in zip(la.get_parameters(), lb.get_parameters()):
            assert np.array_equal(np.asarray(pa), np.asarray(pb))


def test_mlp_recipe_recorded_steps_equal_eager_steps():
    """The recipe has no dropout, so `record_steps` may replay it: the regulariser's sums and gradient terms are kernels of
    the recording.  Same kernels in the same order: losses (data and regularisation), learning rate and parameters
    must agree exactly with the steps launched from Python, replay after replay."""
    import aether

    def make():
        np.random.seed(8)
        m = mlp_model(aether)
        _scaled(m, aether)
        m.loss.new_pass()
        m.accuracy.new_pass()
        return m

    rng = np.random.RandomState(12)
    Xs = [rng.rand(128, 3072).astype(np.float32) for _ in range(2)]
    ys = [rng.randint(0, 10, 128) for _ in range(2)]
    eager, rec = make(), make()
    rec.record_steps(True)
    assert rec.recording_active
    for step in range(6):
        a = eager.train_step(Xs[step % 2], ys[step % 2])
        b = rec.train_step(Xs[step % 2], ys[step % 2])
        assert a == b, "step %d: eager %r, recorded %r" % (step, a, b)
        assert a[2] > 1e-3                                   # the regularisation loss is part of the comparison
        assert eager.optimizer.current_learning_rate == rec.optimizer.current_learning_rate
        for la, lb in zip(eager.trainable_layers, rec.trainable_layers):
            assert np.array_equal(np.asarray(la.weights), np.asarray(lb.weights)), "weights differ after step %d" % step
            assert np.array_equal(np.asarray(la.biases), np.asarray(lb.biases)), "biases differ after step %d" % step
    assert len([r for r in rec._recordings.values() if r.get("graph")]) == 1


def test_mlp_recipe_with_soft_targets_recorded_and_eager():
    """Model.train_step with a 2-D y_true of class probabilities (mixed labels): the loss and the gradients of the first
    step against the oracle, the accuracy from the rows' argmax (CNN_model_cupy.py:384-386), and recorded steps
    bit-identical to eager ones (the recording reads the dense targets from a buffer fed before every replay)."""
    import aether
    from tests import abi

    def make():
        np.random.seed(8)
        m = mlp_model(aether)
        _scaled(m, aether)
        m.loss.new_pass()
        m.accuracy.new_pass()
        return m

    rng = np.random.RandomState(15)
    X = rng.rand(128, 3072).astype(np.float32)
    ys = []
    for _ in range(2):
        a, b = np.eye(10)[rng.randint(0, 10, 128)], np.eye(10)[rng.randint(0, 10, 128)]
        lam = rng.rand(128, 1)
        ys.append((lam * a + (1 - lam) * b).astype(np.float32))
    eager, rec = make(), make()
    net = OracleMlp(host_params(eager))
    rec.record_steps(True)
    for step in range(5):
        y = ys[step % 2]
        before = SC.snapshot(eager)
        a = eager.train_step(X, y)
        b = rec.train_step(X, y)
        assert a == b, "step %d: eager %r, recorded %r" % (step, a, b)
        if step == 0:
            probs, ins, pre = net.forward(X)
            want = float(np.mean(O.cce_forward(probs, y.astype(np.float64), 0.0)))
            assert abs(a[1] - want) <= 1e-5 + 1e-4 * want
            assert a[3] == float(np.mean(np.argmax(probs, axis=1) == np.argmax(y, axis=1)))
            d = O.softmax_cce_backward(probs, y.astype(np.float64), 0.0)
            dw, db, _ = O.dense_backward(ins[-1], net.p[-1][0], net.p[-1][1], d, wl2=WIDTHS[-1][2], bl2=WIDTHS[-1][2],
                                         dtype=np.float64)
            abi.close(eager.trainable_layers[-1].dweights.get(), dw, rms_scaled=True)
        SC.check_update_from_own_state(eager, before, eager.optimizer.current_learning_rate, step)
        for la, lb in zip(eager.trainable_layers, rec.trainable_layers):
            assert np.array_equal(np.asarray(la.weights), np.asarray(lb.weights)), step
    assert len([r for r in rec._recordings.values() if r.get("graph")]) == 1
