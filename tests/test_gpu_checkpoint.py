"""The reference's own trained parameters through the GPU forward pass.

tests/golden/model5_weights.npz holds the 22 arrays of the reference checkpoint
CNN/saved_models/model5, taken out of the pickle stream with pickletools.genops
(tests/golden/make_checkpoint_weights.py: nothing from the file is executed).  Here they
are written back in the reference's CuPy pickle form -- the test first checks that this
file IS the reference's file, byte for byte outside the FRAME opcodes -- and loaded with
Model.load_parameters into the F-MNIST network of CNN/architectures/CNN_test2_cupy.py:31-59.
predict / evaluate on a seeded synthetic batch are compared with the float64 oracle
forward (batch-norm inference path, float64 -> float32 dense weights, (1,1,1,C) running
statistics, NHWC flatten order of Dense-1's rows).

The reference's published accuracies for this checkpoint (CNN_test2_cupy.py:81-88) stay
"parity unpinned": the Fashion-MNIST files are not part of the reference tree.

Tolerance: probabilities within 1e-5 + 1e-3*|oracle| (three convolutions, three batch
norms and two dense layers of float32 rounding against float64)."""
import io
import os
import json

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TUPLES = (2, 4, 2, 4, 2, 4, 2, 2)


def reference_params():
    z = np.load(os.path.join(GOLDEN, "model5_weights.npz"))
    arrays = [z["a%02d" % i] for i in range(22)]
    out, i = [], 0
    for n in TUPLES:
        out.append(tuple(arrays[i:i + n]))
        i += n
    return out


def fmnist_model(aether):
    """CNN/architectures/CNN_test2_cupy.py:29-67."""
    m = aether.Model()
    m.add(aether.Conv_Layer(input_shape=(28, 28, 1), num_filters=32, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Batch_Norm(epsilon=1e-5, momentum=0.9))
    m.add(aether.ReLU())
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Conv_Layer(input_shape=(14, 14, 32), num_filters=64, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Batch_Norm(epsilon=1e-5, momentum=0.9))
    m.add(aether.ReLU())
    m.add(aether.Layer_Dropout_Spatial(rate=0.075))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Conv_Layer(input_shape=(7, 7, 64), num_filters=128, filter_size=(3, 3), strides=(1, 1), padding="same"))
    m.add(aether.Batch_Norm(epsilon=1e-5, momentum=0.9))
    m.add(aether.ReLU())
    m.add(aether.Layer_Dropout_Spatial(rate=0.1))
    m.add(aether.Pooling(filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"))
    m.add(aether.Flatten())
    m.add(aether.Layer_Dense(3 * 3 * 128, n_neurons=256, weight_regularizer_l2=2e-5, bias_regularizer_l2=2e-5))
    m.add(aether.Leaky_ReLU(alpha=0.01))
    m.add(aether.Layer_Dropout(rate=0.075))
    m.add(aether.Layer_Dense(256, 10))
    m.add(aether.SoftMax())
    m.set(loss=aether.Loss_CategoricalCrossEntropy(label_smoothing=0.01),
          optimizer=aether.Optimizer_Adam(learning_rate=0.001, decay=5e-5),
          accuracy=aether.Accuracy_Categorical())
    m.finalize()
    return m


def test_reference_checkpoint_loads_and_predicts_like_the_oracle(tmp_path, capsys):
    import aether
    from aether.model import write_parameters
    from tests import abi
    from tests.test_parameter_files import unframed_sha256
    params = reference_params()
    path = str(tmp_path / "model5")
    write_parameters(params, path, cupy_arrays=True)
    digests = json.load(open(os.path.join(GOLDEN, "checkpoint_digests.json")))["models"]["model5"]
    assert unframed_sha256(open(path, "rb").read()) == digests["unframed_sha256"]     # the reference's file

    np.random.seed(0)
    model = fmnist_model(aether)
    model.load_parameters(path)

    # what went in comes back: float32 arrays exactly, Dense float64 rounded once to float32
    got = model.get_parameters()
    assert [len(t) for t in got] == list(TUPLES)
    for tup, ref in zip(got, params):
        for a, b in zip(tup, ref):
            a = np.asarray(a)
            assert a.dtype == np.float32 and a.size == b.size
            assert np.array_equal(a.reshape(b.shape), b.astype(np.float32))
    for i in (1, 3, 5):                                   # running statistics keep the keepdims shape
        assert np.asarray(got[i][2]).shape == params[i][2].shape == (1, 1, 1, params[i][0].shape[0])
    assert model.layers[0].weights is model.layers[0].filter_weights

    rng = np.random.RandomState(7)
    X = (rng.rand(64, 28, 28, 1).astype(np.float32) * 2 - 1)           # images scaled to [-1, 1] as the script does
    y = rng.randint(0, 10, 64)
    probs = model.predict(X, batch_size=24)                             # 24 + 24 + 16: a ragged last batch
    net = O.OracleCNN([tuple(np.asarray(a, np.float32) for a in t) for t in params], dtype=np.float64)
    want, _ = net.forward(X.astype(np.float64), training=False)
    assert probs.shape == (64, 10)
    abi.close(probs, want, rtol=1e-3)
    assert np.array_equal(np.argmax(probs, axis=1), np.argmax(want, axis=1))
    # the network is trained: it is confident on most of what it sees, not uniform
    assert float(np.mean(np.max(want, axis=1))) > 0.5

    model.evaluate(X, y, batch_size=32)
    line = [l for l in capsys.readouterr().out.splitlines() if l.startswith("Valdiation")][-1]
    loss = float(np.mean(O.cce_forward(want, y, 0.01, training=False)))
    acc = float(np.mean(np.argmax(want, axis=1) == y))
    assert line == f'Valdiation, acc: {acc:.3f}, loss: {loss:.3f}'


def test_loaded_checkpoint_survives_a_save_and_reload(tmp_path):
    import aether
    from aether.model import write_parameters
    params = reference_params()
    path = str(tmp_path / "in")
    write_parameters(params, path, cupy_arrays=True)
    np.random.seed(0)
    a, b = fmnist_model(aether), fmnist_model(aether)
    a.load_parameters(path)
    out = str(tmp_path / "out")
    a.save_parameters(out, cupy_arrays=True)
    b.load_parameters(out)
    X = np.random.RandomState(1).rand(8, 28, 28, 1).astype(np.float32)
    assert np.array_equal(a.predict(X), b.predict(X))
