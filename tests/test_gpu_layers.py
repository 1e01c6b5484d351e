"""Parity of the layer classes (reference API, HIP underneath) with the CPU
oracle.  fp32 tolerance 1e-5 + 1e-4*|oracle| unless a test says otherwise;
index / mask / selection work (pooling argmax, ReLU masks) is bit-exact."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _close(got, want, **kw):
    from tests import abi
    return abi.close(np.asarray(got), want, **kw)


# ---- Conv_Layer class API ---------------------------------------------------------
def test_conv_layer_api_and_parity():
    import aether
    np.random.seed(0)
    layer = aether.Conv_Layer((12, 12, 8), num_filters=16, filter_size=(3, 3), strides=(1, 1), padding="same")
    assert layer.weights is layer.filter_weights
    assert layer.filter_weights.shape == (3, 3, 8, 16) and layer.biases.shape == (16,)
    assert layer.weight_regularizer_l2 == 0 and layer.bias_regularizer_l1 == 0
    # He-normal draw from the legacy global RNG in the reference's order
    np.random.seed(0)
    want_w = np.random.randn(3, 3, 8, 16).astype(np.float32) * np.sqrt(np.float32(2.0 / 72))
    assert np.array_equal(layer.filter_weights.get(), want_w)
    assert np.all(layer.biases.get() == 0)
    x = np.random.randn(4, 12, 12, 8).astype(np.float32)
    dy = np.random.randn(4, 12, 12, 16).astype(np.float32)
    b = np.random.randn(16).astype(np.float32)
    layer.set_parameters(want_w, b)
    assert layer.weights is layer.filter_weights            # alias refreshed
    out = layer.forward(x, training=True)
    assert out is layer.output and out.shape == (4, 12, 12, 16)
    _close(out, O.conv_fprop(x, want_w, b, (1, 1), "same", dtype=np.float64))
    ret = layer.backward(dy)
    assert ret is layer.dinputs and ret.shape == x.shape
    _close(layer.dinputs, O.conv_dgrad(dy, want_w, (12, 12), (1, 1), "same", dtype=np.float64))
    _close(layer.dweights, O.conv_wgrad(x, dy, (3, 3), (1, 1), "same", dtype=np.float64), rms_scaled=True)
    _close(layer.dbiases, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True)
    w2, b2 = layer.get_parameters()
    assert w2 is layer.filter_weights and b2 is layer.biases
    with pytest.raises(ValueError):
        layer.forward(np.zeros((4, 12, 12), np.float32), training=True)


def test_conv_layer_same_with_1x1_returns_full_gradient():
    import aether
    np.random.seed(1)
    layer = aether.Conv_Layer((6, 6, 4), num_filters=8, filter_size=(1, 1), strides=(1, 1), padding="same")
    x = np.random.randn(2, 6, 6, 4).astype(np.float32)
    dy = np.random.randn(2, 6, 6, 8).astype(np.float32)
    layer.forward(x, True)
    layer.backward(dy)
    assert layer.dinputs.shape == (2, 6, 6, 4)
    w = layer.filter_weights.get()
    _close(layer.dinputs, (dy.reshape(-1, 8).astype(np.float64) @ w.reshape(4, 8).T.astype(np.float64)).reshape(2, 6, 6, 4))


# ---- dense ------------------------------------------------------------------------------
@pytest.mark.parametrize("M,n_in,n_out", [(128, 2048, 256), (128, 256, 10), (7, 5, 3), (33, 100, 64)])
def test_dense_parity(M, n_in, n_out):
    import aether
    np.random.seed(2)
    layer = aether.Layer_Dense(n_in, n_out, weight_regularizer_l1=1e-3, bias_regularizer_l1=2e-3,
                               weight_regularizer_l2=3e-3, bias_regularizer_l2=4e-3)
    assert layer.weights.shape == (n_in, n_out) and layer.biases.shape == (1, n_out)
    w = (np.random.randn(n_in, n_out) * 0.1).astype(np.float32)
    w[0, 0] = 0.0                                         # sign(0) = +1 in the L1 term
    b = np.random.randn(1, n_out).astype(np.float32)
    layer.set_parameters(w, b)
    x = np.random.randn(M, n_in).astype(np.float32)
    dy = np.random.randn(M, n_out).astype(np.float32)
    layer.forward(x, training=True)
    # outputs here have rms ~ 0.1*sqrt(n_in) > 1: the absolute part of the
    # tolerance is scaled by that rms (see tests/abi.py)
    _close(layer.output, O.dense_forward(x, w, b, dtype=np.float64), rms_scaled=True)
    assert layer.backward(dy) is None
    dw, db, dx = O.dense_backward(x, w, b, dy, wl1=1e-3, wl2=3e-3, bl1=2e-3, bl2=4e-3, dtype=np.float64)
    _close(layer.dweights, dw, rms_scaled=True)
    _close(layer.dbiases, db, rms_scaled=True)
    _close(layer.dinputs, dx, rms_scaled=True)
    assert layer.dbiases.shape == (1, n_out)


# ---- activations ---------------------------------------------------------------------------
def test_relu_and_leaky_relu_bit_exact():
    import aether
    r = np.random.RandomState(3)
    x = r.randn(5, 7, 3, 9).astype(np.float32)
    x[0, 0, 0, :3] = [0.0, -0.0, 1e-30]
    dy = r.randn(*x.shape).astype(np.float32)
    relu = aether.ReLU()
    relu.forward(x, True)
    relu.backward(dy)
    assert np.array_equal(relu.output.get(), O.relu_forward(x))
    assert np.array_equal(relu.dinputs.get(), O.relu_backward(x, dy))
    lk = aether.Leaky_ReLU(0.01)
    lk.forward(x, True)
    lk.backward(dy)
    assert np.array_equal(lk.output.get(), O.leaky_relu_forward(x, 0.01))
    assert np.array_equal(lk.dinputs.get(), O.leaky_relu_backward(x, dy, 0.01))
    assert aether.Leaky_ReLU().alpha == 0.01


# ---- pooling -----------------------------------------------------------------------------------
def test_maxpool_notebook_example_and_ties():
    import aether
    # CNN/notebooks/Backpropagation_Pooling.ipynb:103-128
    a = np.array([[1, 2, 3, 4], [4, 5, 6, 5], [7, 8, 9, 6], [8, 7, 6, 5]], dtype=np.float32)
    pool = aether.Pooling()
    out = pool.forward(a[None, :, :, None], True)
    assert np.array_equal(out.get()[0, :, :, 0], [[5, 6], [8, 9]])
    pool.backward(out)
    want = np.zeros((4, 4), np.float32)
    want[1, 1], want[1, 2], want[2, 1], want[2, 2] = 5, 6, 8, 9
    assert np.array_equal(pool.dinputs.get()[0, :, :, 0], want)
    # all-zero window (post-ReLU) routes to the top-left element
    z = np.zeros((1, 2, 2, 1), np.float32)
    pool.forward(z, True)
    pool.backward(np.ones((1, 1, 1, 1), np.float32))
    assert np.array_equal(pool.dinputs.get()[0, :, :, 0], [[1, 0], [0, 0]])


@pytest.mark.parametrize("shape,f,s", [((4, 16, 16, 32), (2, 2), (2, 2)), ((2, 7, 6, 3), (2, 2), (2, 2)),
                                       ((2, 9, 9, 5), (3, 3), (2, 2)), ((2, 8, 8, 4), (2, 2), (1, 1)),
                                       ((3, 10, 7, 6), (3, 2), (1, 2)), ((2, 9, 10, 8), (3, 3), (2, 2)),
                                       ((2, 11, 7, 12), (3, 2), (1, 1))])
def test_maxpool_bit_exact(shape, f, s):
    import aether
    r = np.random.RandomState(4)
    x = r.randint(0, 5, shape).astype(np.float32)          # many ties
    pool = aether.Pooling(filter_size=f, strides=s)
    pool.forward(x, True)
    pooled, idx = O.maxpool_forward(x, f, s)
    assert np.array_equal(pool.output.get(), pooled)
    assert np.array_equal(pool.max_indicies.get(), idx.astype(np.uint8))
    dy = r.randn(*pooled.shape).astype(np.float32)
    pool.backward(dy)
    want = O.maxpool_backward(dy, idx, x.shape, f, s)
    if s[0] >= f[0] and s[1] >= f[1]:
        assert np.array_equal(pool.dinputs.get(), want)
    else:
        _close(pool.dinputs, want)


def test_avgpool_and_pooling_errors():
    import aether
    a = np.array([[1, 2, 3, 4], [4, 5, 6, 5], [7, 8, 9, 6], [8, 7, 6, 5]], dtype=np.float32)
    pool = aether.Pooling(pooling_type="average")
    out = pool.forward(a[None, :, :, None], True)
    assert np.array_equal(out.get()[0, :, :, 0], [[3, 4.5], [7.5, 6.5]])      # nb :483-516
    pool.backward(out)
    assert np.array_equal(pool.dinputs.get()[0, :2, 2:, 0], np.full((2, 2), 1.125))
    r = np.random.RandomState(5)
    x = r.randn(2, 9, 8, 3).astype(np.float32)
    pool = aether.Pooling((3, 3), (2, 1), pooling_type="average")
    pool.forward(x, True)
    _close(pool.output, O.avgpool_forward(x, (3, 3), (2, 1)))
    dy = r.randn(*pool.output.shape).astype(np.float32)
    pool.backward(dy)
    _close(pool.dinputs, O.avgpool_backward(dy, x.shape, (3, 3), (2, 1)))
    # channel counts that are multiples of 4 take 16-byte loads and stores: same sums
    for shape, f, s in (((2, 9, 8, 8), (3, 3), (2, 1)), ((3, 8, 6, 12), (2, 2), (2, 2)), ((2, 7, 7, 4), (2, 3), (1, 1))):
        x = r.randn(*shape).astype(np.float32)
        pool = aether.Pooling(f, s, pooling_type="average")
        pool.forward(x, True)
        _close(pool.output, O.avgpool_forward(x, f, s))
        dy = r.randn(*pool.output.shape).astype(np.float32)
        pool.backward(dy)
        _close(pool.dinputs, O.avgpool_backward(dy, x.shape, f, s))
    with pytest.raises(ValueError):
        aether.Pooling().forward(np.zeros((2, 4, 4), np.float32), True)
    with pytest.raises(ValueError):
        aether.Pooling(padding="full").forward(np.zeros((2, 4, 4, 1), np.float32), True)


# ---- batch norm ---------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(128, 32, 32, 32), (16, 8, 8, 128), (6, 5, 5, 3), (64, 40), (3, 4, 4, 70)])
def test_batch_norm_parity(shape):
    import aether
    r = np.random.RandomState(6)
    C = shape[-1]
    x = (r.randn(*shape) * 2 + 5).astype(np.float32)       # mean >> 0 stresses the variance
    dy = r.randn(*shape).astype(np.float32)
    g = (r.rand(C) + 0.5).astype(np.float32)
    be = r.randn(C).astype(np.float32)
    bn = aether.Batch_Norm()
    assert bn.gamma is None and bn.running_mean is None
    bn.forward(x, training=True)                            # lazy init: gamma 1, beta 0
    assert np.all(bn.gamma.get() == 1) and np.all(bn.beta.get() == 0)
    assert bn.weights is bn.gamma and bn.biases is bn.beta
    bn.set_parameters(g, be, np.zeros(C, np.float32), np.ones(C, np.float32))
    bn.forward(x, training=True)
    x64 = x.astype(np.float64)
    y, xhat, mu, var, rm, rv = O.bn_forward_train(x64, g.astype(np.float64), be.astype(np.float64),
                                                  np.zeros(C), np.ones(C), 1e-5, 0.9)
    _close(bn.output, y)
    assert bn.running_mean.shape == rm.shape               # keepdims shape, as saved by the reference
    _close(bn.running_mean, rm)
    _close(bn.running_var, rv)
    bn.backward(dy)
    dx, dg, db = O.bn_backward(x64, dy.astype(np.float64), g.astype(np.float64), mu, var, 1e-5)
    _close(bn.dinputs, dx)
    _close(bn.dweights, dg, rms_scaled=True)
    _close(bn.dbiases, db, rms_scaled=True)
    bn.forward(x, training=False)
    _close(bn.output, O.bn_forward_infer(x64, g.astype(np.float64), be.astype(np.float64), rm, rv, 1e-5))
    assert len(bn.get_parameters()) == 4


# ---- dropout -------------------------------------------------------------------------------------
def test_dropout_layers_with_reference_shaped_masks():
    import aether
    r = np.random.RandomState(7)
    x = r.randn(4, 6, 6, 8).astype(np.float32)
    dy = r.randn(*x.shape).astype(np.float32)
    d = aether.Layer_Dropout(0.25)
    assert d.rate == 0.75
    np.random.seed(11)
    d.forward(x, training=True)
    np.random.seed(11)
    mask = (np.random.binomial(1, 0.75, size=x.shape) / 0.75).astype(np.float32)
    assert np.array_equal(d.output.get(), mask * x)
    d.backward(dy)
    assert np.array_equal(d.dinputs.get(), dy * mask)
    d.forward(x, training=False)
    assert np.array_equal(d.output.get(), x)
    sp = aether.Layer_Dropout_Spatial(0.5)
    np.random.seed(12)
    sp.forward(x, training=True)
    np.random.seed(12)
    cmask = (np.random.binomial(1, 0.5, size=(1, 1, 1, 8)) / 0.5).astype(np.float32)
    assert np.array_equal(sp.output.get(), x * cmask)
    sp.backward(dy)
    assert np.array_equal(sp.dinputs.get(), dy * cmask)
    d0 = aether.Layer_Dropout(0.0)                           # rate 0: identity
    d0.forward(x, training=True)
    assert np.array_equal(d0.output.get(), x)


# ---- flatten / softmax / loss / adam ------------------------------------------------------------------
def test_flatten_softmax_loss():
    import aether
    r = np.random.RandomState(8)
    x = r.randn(4, 3, 2, 5).astype(np.float32)
    fl = aether.Flatten()
    fl.forward(x, True)
    assert np.array_equal(fl.output.get(), x.reshape(4, -1))
    fl.backward(fl.output)
    assert fl.dinputs.shape == x.shape
    logits = (r.randn(128, 10) * 3).astype(np.float32)
    y = r.randint(0, 10, 128)
    sm = aether.SoftMax()
    sm.forward(logits, True)
    p64 = O.softmax(logits.astype(np.float64))
    _close(sm.output, p64)
    assert np.array_equal(sm.predictions(sm.output), np.argmax(p64, axis=1))
    dv = r.randn(128, 10).astype(np.float32)
    sm.backward(dv)
    jac = np.stack([(np.diagflat(p) - np.outer(p, p)) @ d for p, d in zip(p64, dv.astype(np.float64))])
    _close(sm.dinputs, jac)
    for ls in (0.0, 0.01):
        loss = aether.Loss_CategoricalCrossEntropy(label_smoothing=ls)
        loss.new_pass()
        loss.remember_trainable_layers([])
        data_loss, reg = loss.calculate(sm.output, y, include_regularization=True, training=True)
        want = O.cce_forward(p64, y, ls, training=True)
        assert abs(data_loss - want.mean()) <= 1e-5 + 1e-4 * abs(want.mean()) and reg == 0
        ev = loss.calculate(sm.output, y, training=False)
        assert abs(ev - O.cce_forward(p64, y, ls, training=False).mean()) <= 1e-4
        assert abs(loss.calculate_accumulated() - (want.sum() + O.cce_forward(p64, y, 0.0).sum()) / 256) <= 1e-4
        comb = aether.Activation_Softmax_Loss_CategoricalCrossEntropy(ls)
        comb.backward(sm.output, y, training=True)
        _close(comb.dinputs, O.softmax_cce_backward(p64, y, ls))
        comb.backward(sm.output, np.eye(10)[y], training=True)        # one-hot labels
        _close(comb.dinputs, O.softmax_cce_backward(p64, y, ls))


@pytest.mark.parametrize("K", [10, 16, 37])
def test_soft_targets(K):
    """2-D targets that are not one-hot (CNN_classes_cupy.py:622-626, :672-676 use them as given): the loss, both
    backward forms and the one-launch head take dense rows; one-hot rows handed in as dense rows give the very
    bits of the index form."""
    import aether
    from aether import _lib
    from aether.tensor import DeviceTensor
    r = np.random.RandomState(18)
    S = 77
    logits = (r.randn(S, K) * 3).astype(np.float32)
    t = (r.rand(S, K) ** 3).astype(np.float32)
    t /= t.sum(axis=1, keepdims=True)
    p64 = O.softmax(logits.astype(np.float64))
    sm = aether.SoftMax()
    sm.forward(logits, True)
    for ls in (0.0, 0.05):
        loss = aether.Loss_CategoricalCrossEntropy(label_smoothing=ls)
        loss.new_pass()
        loss.remember_trainable_layers([])
        per_sample = loss.forward(sm.output, t, training=True)
        _close(per_sample, O.cce_forward(p64, t.astype(np.float64), ls, training=True))
        _close(loss.forward(sm.output, t, training=False), O.cce_forward(p64, t.astype(np.float64), ls, training=False))
        assert np.array_equal(sm.predictions(sm.output), np.argmax(p64, axis=1))
        want = O.softmax_cce_backward(p64, t.astype(np.float64), ls)
        comb = aether.Activation_Softmax_Loss_CategoricalCrossEntropy(ls)
        comb.backward(sm.output, t, training=True)
        _close(comb.dinputs, want)
        loss.backward(sm.output, t)
        _close(loss.dinputs, want)
        # the head of a training step in one launch
        head, fused = aether.SoftMax(), aether.Activation_Softmax_Loss_CategoricalCrossEntropy(ls)
        pending = loss.head_launch(DeviceTensor.from_numpy(logits), t, head, fused)
        _close(loss.forward_finish(pending), O.cce_forward(p64, t.astype(np.float64), ls, training=True))
        assert np.array_equal(head.output.get(), sm.output.get())
        assert np.array_equal(fused.dinputs.get(), comb.dinputs.get())
    # one-hot rows through the dense entry points == the index entry points, bit for bit
    L = _lib.lib()
    y = r.randint(0, K, S).astype(np.int32)
    lg, yd, td = DeviceTensor.from_numpy(logits), DeviceTensor.from_numpy(y, np.int32), DeviceTensor.from_numpy(np.eye(K, dtype=np.float32)[y])
    outs = []
    for fn, tg in ((L.aeth_softmax_cce_train_f32, yd), (L.aeth_softmax_cce_train_dense_f32, td)):
        probs, buf, dl = DeviceTensor.full((S, K), np.nan), DeviceTensor.full(2 * S, np.nan), DeviceTensor.full((S, K), np.nan)
        _lib.check(fn(lg.ptr, tg.ptr, 0.1, probs.ptr, buf.ptr, buf.ptr + 4 * S, dl.ptr, S, K))
        outs.append((probs.get(), buf.get(), dl.get()))
    assert all(np.array_equal(a, b) for a, b in zip(*outs))
    assert L.aeth_cce_fwd_dense_f32(lg.ptr, None, 0.0, lg.ptr, lg.ptr, S, K) == _lib.AETH_E_INVALID


@pytest.mark.parametrize("n", [1, 1000, 16384, 16385, 100001, 786432, 5000003])
def test_sums_for_the_regularisers(n):
    """aeth_reduce_f32 (sum |x| and sum x^2 behind Loss.regularization_loss, CNN_classes_cupy.py:593-609): one block
    for short inputs, chunks and a second stage for long ones; the same bits on every call."""
    import ctypes as C
    import aether
    from aether import _lib
    L = _lib.lib()
    x = np.random.RandomState(n % 1000).randn(n).astype(np.float32)
    xd = aether.DeviceTensor.from_numpy(x)
    out = aether.DeviceTensor.zeros(1)
    for mode, want in ((0, np.abs(x.astype(np.float64)).sum()), (1, (x.astype(np.float64) ** 2).sum())):
        _lib.check(L.aeth_reduce_f32(xd.ptr, C.c_int64(n), mode, out.ptr))
        got = float(out.get()[0])
        assert abs(got - want) <= 2e-6 * want + 1e-30, (n, mode, got, want)
        _lib.check(L.aeth_reduce_f32(xd.ptr, C.c_int64(n), mode, out.ptr))
        assert float(out.get()[0]) == got


def test_regularization_loss_and_adam():
    import aether
    np.random.seed(9)
    dense = aether.Layer_Dense(20, 30, weight_regularizer_l1=0.1, bias_regularizer_l1=0.2,
                               weight_regularizer_l2=0.3, bias_regularizer_l2=0.4)
    w = np.random.randn(20, 30).astype(np.float32)
    b = np.random.randn(1, 30).astype(np.float32)
    dense.set_parameters(w, b)
    loss = aether.Loss_CategoricalCrossEntropy()
    loss.remember_trainable_layers([dense])
    want = 0.1 * np.abs(w).sum() + 0.3 * (w * w).sum() + 0.2 * np.abs(b).sum() + 0.4 * (b * b).sum()
    assert abs(loss.regularization_loss() - want) <= 1e-4 * want
    opt = aether.Optimizer_Adam(learning_rate=1e-3, decay=1e-2)
    th, bb = w.astype(np.float64), b.astype(np.float64)
    m = [np.zeros_like(th), np.zeros_like(bb)]
    v = [np.zeros_like(th), np.zeros_like(bb)]
    for it in range(4):
        gw = np.random.randn(20, 30).astype(np.float32)
        gb = np.random.randn(1, 30).astype(np.float32)
        dense.dweights = aether.DeviceTensor.from_numpy(gw)
        dense.dbiases = aether.DeviceTensor.from_numpy(gb)
        opt.pre_update_parameters()
        opt.update_parameters(dense)
        opt.post_update_parameters()
        lr = 1e-3 / (1 + 1e-2 * it)
        assert abs(opt.current_learning_rate - lr) < 1e-12
        th, m[0], v[0] = O.adam_update(th, gw.astype(np.float64), m[0], v[0], lr, it)
        bb, m[1], v[1] = O.adam_update(bb, gb.astype(np.float64), m[1], v[1], lr, it)
        _close(dense.weights, th)
        _close(dense.biases, bb)
    assert opt.iterations == 4
    _close(dense.weight_momentums, m[0])
    _close(dense.weight_cache, v[0], atol=1e-7)


def _block(aether, alpha):
    """Batch_Norm -> activation -> Pooling wired the way Model.finalize wires them."""
    bn = aether.Batch_Norm()
    act = aether.ReLU() if alpha is None else aether.Leaky_ReLU(alpha=alpha)
    pool = aether.Pooling()
    bn.next, act.next = act, pool
    return bn, act, pool


@pytest.mark.parametrize("shape,alpha", [((8, 16, 16, 32), None), ((3, 6, 10, 8), 0.01), ((5, 4, 2, 64), None),
                                         ((2, 7, 6, 8), None), ((2, 6, 6, 6), None), ((2, 4, 4, 24), 0.2)])
def test_fused_block_equals_the_three_layers(shape, alpha, monkeypatch):
    import aether
    r = np.random.RandomState(5)
    x = (r.randn(*shape) * 2.0 + 0.5).astype(np.float32)
    x[0, :2, :2, 0] = 1.25                      # a window of equal values: the first one wins the pooling
    dy = r.randn(shape[0], shape[1] // 2, shape[2] // 2, shape[3]).astype(np.float32)
    got = {}
    for fuse in ("1", "0"):
        monkeypatch.setenv("AETHER_FUSE_BLOCK", fuse)
        bn, act, pool = _block(aether, alpha)
        bn.forward(x, True)
        act.forward(bn.output, True)
        pool.forward(act.output, True)
        pool.backward(dy)
        act.backward(pool.dinputs)
        bn.backward(act.dinputs)
        got[fuse] = [t.get() for t in (bn.output, act.output, pool.output, pool.max_indicies, pool.dinputs,
                                       act.dinputs, bn.dinputs, bn.dweights, bn.dbiases, bn.running_mean,
                                       bn.running_var)]
        fused_ran = getattr(pool, "_fused_relu", None) is not None
        even = shape[1] % 2 == 0 and shape[2] % 2 == 0 and shape[3] % 4 == 0
        assert fused_ran == (fuse == "1" and even)
    for a, b in zip(got["1"], got["0"]):
        assert a.shape == b.shape
        # the column sums of the batch norm's backward pass are added in another order
        assert np.allclose(a, b, rtol=2e-5, atol=2e-5 * max(1.0, float(np.abs(b).max())))
    # the indices agree exactly wherever the activations do
    same = np.all(got["1"][1] == got["0"][1])
    assert not same or np.array_equal(got["1"][3], got["0"][3])


@pytest.mark.parametrize("M,n_in,n_mid,n_out,alpha", [(128, 2048, 256, 10, 0.01), (128, 2048, 256, 10, None), (37, 300, 64, 16, 0.2),
                                                       (64, 512, 128, 40, None), (5, 24, 8, 3, 0.1), (1100, 96, 32, 10, None)])
def test_dense_layers_with_the_activation_next_to_them(M, n_in, n_mid, n_out, alpha, monkeypatch):
    """Layer_Dense -> ReLU / Leaky_ReLU -> Layer_Dense: the first layer's forward call also writes the activation's output
    (from the reduction of its split K where there is one), the second layer's backward call is one launch for a layer of
    at most 16 outputs and also does the activation's backward pass.  The same values as layer by layer
    (AETHER_FUSE_DENSE=0), bit for bit, and the oracle's."""
    import aether
    r = np.random.RandomState(19)
    x = r.randn(M, n_in).astype(np.float32)
    dy = r.randn(M, n_out).astype(np.float32)
    w1, b1 = (r.randn(n_in, n_mid) / np.sqrt(n_in)).astype(np.float32), r.randn(1, n_mid).astype(np.float32)
    w2, b2 = (r.randn(n_mid, n_out) / np.sqrt(n_mid)).astype(np.float32), r.randn(1, n_out).astype(np.float32)
    got = {}
    for fuse in ("1", "0"):
        monkeypatch.setenv("AETHER_FUSE_DENSE", fuse)
        d1, d2 = aether.Layer_Dense(n_in, n_mid), aether.Layer_Dense(n_mid, n_out, weight_regularizer_l2=1e-3)
        act = aether.ReLU() if alpha is None else aether.Leaky_ReLU(alpha)
        d1.set_parameters(w1, b1)
        d2.set_parameters(w2, b2)
        d1.next, act.prev, act.next, d2.prev = act, d1, d2, act       # as Model.finalize links them
        d1.forward(x, True)
        act.forward(d1.output, True)
        d2.forward(act.output, True)
        d2.backward(dy)
        act.backward(d2.dinputs)
        d1.backward(act.dinputs)
        got[fuse] = [t.get() for t in (d1.output, act.output, d2.output, d2.dweights, d2.dbiases, d2.dinputs, act.dinputs,
                                       d1.dweights, d1.dbiases, d1.dinputs)]
        assert (getattr(act, "_prefilled_for", None) is None) and (getattr(act, "_bwd_prefilled_for", None) is None)
    for a, b in zip(got["1"], got["0"]):
        assert np.array_equal(a, b)
    a64 = alpha if alpha is not None else 0.0
    y1 = O.dense_forward(x, w1, b1, dtype=np.float64)
    h = np.where(y1 > 0, y1, a64 * y1)
    _close(got["1"][0], y1)
    _close(got["1"][1], h)
    dw2, db2, dh = O.dense_backward(h, w2, b2, dy, wl2=1e-3, dtype=np.float64)
    _close(got["1"][3], dw2, rms_scaled=True)
    _close(got["1"][4], db2, rms_scaled=True)
    _close(got["1"][5], dh)
    # the activation's gradient follows the sign of ITS input as the GPU saw it (float32 y1)
    _close(got["1"][6], np.where(got["1"][0] < 0, a64 * dh, dh))


def test_fused_block_entry_points_reject_what_they_do_not_cover():
    from aether import _lib
    from aether.tensor import DeviceTensor
    L = _lib.lib()
    t = DeviceTensor.zeros(4 * 4 * 4 * 8)
    c = DeviceTensor.zeros(8)
    i8 = DeviceTensor((4 * 2 * 2 * 8,), np.uint8)
    args = (t.ptr, c.ptr, c.ptr, c.ptr, c.ptr, c.ptr, c.ptr, t.ptr, t.ptr, t.ptr, i8.ptr)
    assert L.aeth_bn_relu_maxpool2_fwd_f32(*args, 4, 3, 4, 8, 1e-5, 0.9, 0.0) == _lib.AETH_E_INVALID     # odd H
    assert L.aeth_bn_relu_maxpool2_fwd_f32(*args, 4, 4, 4, 6, 1e-5, 0.9, 0.0) == _lib.AETH_E_INVALID     # C % 4
    assert L.aeth_maxpool2_relu_bwd_f32(t.ptr, i8.ptr, t.ptr, t.ptr, t.ptr, 4, 4, 5, 8, 0.0) == _lib.AETH_E_INVALID
    assert L.aeth_maxpool2_relu_bwd_f32(None, i8.ptr, t.ptr, t.ptr, t.ptr, 4, 4, 4, 8, 0.0) == _lib.AETH_E_INVALID
    assert L.aeth_bn_relu_maxpool2_fwd_f32(*args, 4, 4, 4, 8, 1e-5, 0.9, 0.0) == 0
    # with the optional bfloat16 copy of the pooling output: the cast of what was written
    from oracle import oracle as O
    r = np.random.RandomState(0)
    t.set(r.randn(t.size))
    pool = DeviceTensor.full(4 * 2 * 2 * 8, np.nan)
    p16 = DeviceTensor(4 * 2 * 2 * 8, np.uint16)
    g, rv = DeviceTensor.full(8, 1.0), DeviceTensor.full(8, 1.0)
    rm, sm, si = DeviceTensor.zeros(8), DeviceTensor.zeros(8), DeviceTensor.zeros(8)
    bn_out, relu_out = DeviceTensor(t.size), DeviceTensor(t.size)
    args2 = (t.ptr, g.ptr, c.ptr, rm.ptr, rv.ptr, sm.ptr, si.ptr, bn_out.ptr, relu_out.ptr, pool.ptr, p16.ptr, i8.ptr)
    assert L.aeth_bn_relu_maxpool2_fwd_twin_f32(*args2, 4, 4, 4, 8, 1e-5, 0.9, 0.0) == 0
    assert np.all(np.isfinite(pool.get())) and np.array_equal(p16.get(), O.bf16_bits(pool.get()))
    args3 = args2[:10] + (None,) + args2[11:]
    assert L.aeth_bn_relu_maxpool2_fwd_twin_f32(*args3, 4, 4, 4, 8, 1e-5, 0.9, 0.0) == _lib.AETH_E_INVALID   # the copy is the point



@pytest.mark.parametrize("nbytes", [4, 65536, 262144 - 4, 262144, 262144 + 4, 1572864, 2097152, 2097152 + 4, 5000000])
def test_host_copies_through_the_staging_slots(nbytes):
    """aeth_memcpy_h2d sends up to 2 MB through pinned slots of 256 KB, piece by piece, and returns at once; the
    source may be overwritten right after the call.  Sizes around a slot, around all 8 slots, and beyond."""
    import aether
    r = np.random.RandomState(nbytes % 977)
    n = nbytes // 4
    src = r.randint(0, 1 << 30, n).astype(np.int32)
    want = src.copy()
    t = aether.DeviceTensor((n,), dtype=np.int32)
    t.set(src)
    src[:] = -1                                    # the call has taken its copy
    again = aether.DeviceTensor.from_numpy(want)   # a second copy queued behind the first: slots are reused in order
    assert np.array_equal(t.get(), want)
    assert np.array_equal(again.get(), want)
