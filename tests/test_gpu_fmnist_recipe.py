"""Whole training steps of the reference's Fashion-MNIST NumPy recipe
(CNN/architectures/CNN_test.py:28-52) on the GPU against the float64 oracle:
Conv(8)-LeakyReLU(0.05)-MaxPool, Conv(16)-LeakyReLU(0.05)-SpatialDropout(0.1)-MaxPool,
Conv(32)-ReLU-SpatialDropout(0.15)-AveragePool, Flatten, Dense(288,256; L2 5e-5 on weights
and biases)-ReLU, Dense(256,10), SoftMax + Loss_CategoricalCrossEntropy() (no smoothing),
Adam(lr 1e-3, decay 1e-5).

No batch norm, 1 / 8 / 16 input channels, a leaky ReLU in front of a max pooling, average
pooling in the last block: the layers the three-block CIFAR network does not combine.
The oracle side composes the pinned primitives of oracle/oracle.py in the order of the
reference's Model.forward / Model.backward (CNN_model.py:153-208); masks are drawn on the
host with the reference's shape ((1,1,1,C)/keep, CNN_classes.py:397-398) and handed to
both sides."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import step_checks as SC
from tests.test_gpu_model import host_params, outside_share, rel_l2

pytestmark = pytest.mark.gpu

L2 = 5e-5
LR, DECAY = 1e-3, 1e-5


def fmnist_model(aether):
    m = aether.Model()
    m.add(aether.Conv_Layer(input_shape=(28, 28, 1), num_filters=8, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Leaky_ReLU(alpha=0.05))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Conv_Layer(input_shape=(14, 14, 8), num_filters=16, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Leaky_ReLU(alpha=0.05))
    m.add(aether.Layer_Dropout_Spatial(rate=0.1))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Conv_Layer(input_shape=(7, 7, 16), num_filters=32, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.ReLU())
    m.add(aether.Layer_Dropout_Spatial(rate=0.15))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="average"))
    m.add(aether.Flatten())
    m.add(aether.Layer_Dense(3 * 3 * 32, n_neurons=256, weight_regularizer_l2=L2, bias_regularizer_l2=L2))
    m.add(aether.ReLU())
    m.add(aether.Layer_Dense(256, 10))
    m.add(aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(),
          optimizer=aether.Optimizer_Adam(learning_rate=LR, decay=DECAY),
          accuracy=aether.Accuracy_Categorical())
    m.finalize()
    return m


class OracleFmnist:
    """The same network from oracle primitives, float64.  ``p``: [conv W,b] x 3, [dense W,b] x 2."""

    def __init__(self, params):
        self.p = [[np.array(a, dtype=np.float64) for a in tup] for tup in params]
        self.m = [[np.zeros_like(a) for a in tup] for tup in self.p]
        self.v = [[np.zeros_like(a) for a in tup] for tup in self.p]
        self.iterations = 0

    def forward(self, X, masks=None):
        dt = np.float64
        masks = masks or {}
        c = {}
        a = np.asarray(X, dtype=dt)
        for blk in range(3):
            W, b = self.p[blk]
            c["conv%d_in" % blk] = a
            a = O.conv_fprop(a, W, b, (1, 1), "same", dtype=dt)
            c["act%d_in" % blk] = a
            a = O.leaky_relu_forward(a, 0.05) if blk < 2 else O.relu_forward(a)
            mask = masks.get("spatial%d" % blk)
            c["mask%d" % blk] = mask
            if mask is not None:
                a = O.dropout_forward(a, np.asarray(mask, dtype=dt).reshape(1, 1, 1, -1))
            c["pool%d_in_shape" % blk] = a.shape
            if blk < 2:
                a, idx = O.maxpool_forward(a, dtype=dt)
                c["pool%d_idx" % blk] = idx
            else:
                a = O.avgpool_forward(a)
        c["flat_shape"] = a.shape
        a = a.reshape(a.shape[0], -1)
        c["d0_in"] = a
        a = O.dense_forward(a, self.p[3][0], self.p[3][1], dtype=dt)
        c["relu_in"] = a
        a = O.relu_forward(a)
        c["d1_in"] = a
        a = O.dense_forward(a, self.p[4][0], self.p[4][1], dtype=dt)
        return O.softmax(a), c

    def step(self, X, y, masks):
        dt = np.float64
        probs, c = self.forward(X, masks)
        loss = float(np.mean(O.cce_forward(probs, y, 0.0, training=True)))
        reg = O.regularization_loss(self.p[3][0], self.p[3][1], wl2=L2, bl2=L2)
        acc = float(np.mean(np.argmax(probs, axis=1) == y))
        grads = [None] * 5
        d = O.softmax_cce_backward(probs, y, 0.0)
        dw, db, d = O.dense_backward(c["d1_in"], self.p[4][0], self.p[4][1], d, dtype=dt)
        grads[4] = (dw, db)
        d = O.relu_backward(c["relu_in"], d)
        dw, db, d = O.dense_backward(c["d0_in"], self.p[3][0], self.p[3][1], d, wl2=L2, bl2=L2, dtype=dt)
        grads[3] = (dw, db)
        d = d.reshape(c["flat_shape"])
        dinputs = {}
        for blk in (2, 1, 0):
            shp = c["pool%d_in_shape" % blk]
            if blk < 2:
                d = O.maxpool_backward(d, c["pool%d_idx" % blk], shp, dtype=dt)
            else:
                d = O.avgpool_backward(d, shp)
            if c["mask%d" % blk] is not None:
                d = O.dropout_backward(d, np.asarray(c["mask%d" % blk], dtype=dt).reshape(1, 1, 1, -1))
            if blk < 2:
                d = O.leaky_relu_backward(c["act%d_in" % blk], d, 0.05)
            else:
                d = O.relu_backward(c["act%d_in" % blk], d)
            W, b = self.p[blk]
            xin = c["conv%d_in" % blk]
            grads[blk] = (O.conv_wgrad(xin, d, W.shape[:2], (1, 1), "same", dtype=dt), O.conv_dbias(d, dtype=dt))
            d = O.conv_dgrad(d, W, xin.shape[1:3], (1, 1), "same", dtype=dt)
            dinputs[blk] = d
        lr = LR * (1.0 / (1.0 + DECAY * self.iterations))
        for i, tup in enumerate(self.p):
            for j in range(2):
                g = np.asarray(grads[i][j]).reshape(tup[j].shape)
                self.p[i][j], self.m[i][j], self.v[i][j] = O.adam_update(tup[j], g, self.m[i][j], self.v[i][j], lr,
                                                                         self.iterations)
        self.iterations += 1
        return {"loss": loss, "reg_loss": reg, "acc": acc, "probs": probs, "grads": grads, "dinputs": dinputs, "lr": lr}


def draw_masks(rng):
    return {"spatial1": (rng.binomial(1, 1 - 0.1, size=(1, 1, 1, 16)) / (1 - 0.1)).astype(np.float32),
            "spatial2": (rng.binomial(1, 1 - 0.15, size=(1, 1, 1, 32)) / (1 - 0.15)).astype(np.float32)}


def test_fmnist_numpy_recipe_steps_match_oracle():
    import aether
    from tests import abi
    np.random.seed(3)
    S = 64
    X = ((np.random.randint(0, 256, size=(S, 28, 28, 1)).astype(np.float32) - 127.5) / 127.5)   # CNN_test.py:23
    y = np.random.randint(0, 10, S)
    model = fmnist_model(aether)
    # Dense-1's fresh weights are ~1e-3 (the reference's 0.01 factor): scale them so that the L2 terms matter
    d1 = [l for l in model.layers if isinstance(l, aether.Layer_Dense)][0]
    d1.set_parameters(np.asarray(d1.weights) * 100, np.full((1, 256), 0.5, np.float32))
    spatial = [l for l in model.layers if isinstance(l, aether.Layer_Dropout_Spatial)]
    params = host_params(model)
    assert [len(t) for t in params] == [2, 2, 2, 2, 2]
    net = OracleFmnist(params)

    model.loss.new_pass()
    model.accuracy.new_pass()
    rng = np.random.RandomState(11)
    for step in range(3):
        masks = draw_masks(rng)
        spatial[0].fixed_mask, spatial[1].fixed_mask = masks["spatial1"], masks["spatial2"]
        before = SC.snapshot(model)
        ref = net.step(X, y, masks)
        loss, data_loss, reg_loss, acc = model.train_step(X, y)
        assert ref["reg_loss"] > 1e-3
        assert abs(data_loss - ref["loss"]) <= 1e-5 + 1e-4 * abs(ref["loss"]), (step, data_loss, ref["loss"])
        assert abs(reg_loss - ref["reg_loss"]) <= 1e-6 + 1e-4 * ref["reg_loss"], (step, reg_loss, ref["reg_loss"])
        assert abs(loss - (ref["loss"] + ref["reg_loss"])) <= 2e-5 + 1e-4 * abs(loss)
        assert abs(acc - ref["acc"]) <= 1.0 / S + 1e-9
        assert model.optimizer.current_learning_rate == pytest.approx(ref["lr"], rel=1e-12)
        assert np.array_equal(spatial[0].channel_mask.get(), masks["spatial1"])
        assert np.array_equal(spatial[1].channel_mask.get(), masks["spatial2"])
        probs = model.layers[-1].output.get()
        assert rel_l2(probs, ref["probs"]) <= (1e-4 if step == 0 else 2e-3)
        if step == 0:
            abi.close(probs, ref["probs"])
            for i, layer in enumerate(model.trainable_layers):
                gw, gb = ref["grads"][i]
                name = "%d:%s" % (i, type(layer).__name__)
                assert rel_l2(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 2e-4, name
                assert outside_share(layer.dweights.get(), gw.reshape(layer.dweights.shape)) <= 1e-3, name
                assert rel_l2(layer.dbiases.get(), gb.reshape(layer.dbiases.shape)) <= 2e-4, name
            # Dense-1's gradients carry 2*lambda*W and 2*lambda*b
            gw, gb = ref["grads"][3]
            assert rel_l2(gw - 2 * L2 * params[3][0].astype(np.float64), gw) > 1e-3
            assert rel_l2(gb - 2 * L2 * params[3][1].astype(np.float64).reshape(gb.shape), gb) > 1e-6
            convs = [l for l in model.layers if isinstance(l, aether.Conv_Layer)]
            for blk, conv in enumerate(convs):
                want = ref["dinputs"][blk]
                assert rel_l2(conv.dinputs.get(), want) <= 2e-4, blk
                assert outside_share(conv.dinputs.get(), want) <= 1e-3, blk
        SC.check_update_from_own_state(model, before, ref["lr"], step)
        if step == 0:
            SC.check_update_against_oracle(model, before, net.p, ref["grads"], ref["lr"])
    assert model.optimizer.iterations == 3

    # evaluation: the dropout layers pass their input through
    probs_eval, _ = net.forward(X, masks=None)
    pred = model.predict(X, batch_size=32)
    assert rel_l2(pred, probs_eval) <= 5e-3
