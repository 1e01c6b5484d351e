"""Pins the supporting-layer part of the CPU oracle: notebook examples, torch
CPU routines of the same formula, closed forms and invariants."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import oracle as O


# ---- pooling -------------------------------------------------------------------
def test_notebook_maxpool_4x4():
    # CNN/notebooks/Backpropagation_Pooling.ipynb:103-128
    a = np.array([[1, 2, 3, 4], [4, 5, 6, 5], [7, 8, 9, 6], [8, 7, 6, 5]], dtype=np.float32)
    pooled, idx = O.maxpool_forward(a[None, :, :, None])
    assert np.array_equal(pooled[0, :, :, 0], [[5, 6], [8, 9]])
    dx = O.maxpool_backward(pooled, idx, (1, 4, 4, 1))
    want = np.zeros((4, 4), dtype=np.float32)
    want[1, 1], want[1, 2], want[2, 1], want[2, 2] = 5, 6, 8, 9
    assert np.array_equal(dx[0, :, :, 0], want)


def test_notebook_avgpool_4x4():
    # Backpropagation_Pooling.ipynb:483-516
    a = np.array([[1, 2, 3, 4], [4, 5, 6, 5], [7, 8, 9, 6], [8, 7, 6, 5]], dtype=np.float32)
    pooled = O.avgpool_forward(a[None, :, :, None])
    assert np.array_equal(pooled[0, :, :, 0], [[3, 4.5], [7.5, 6.5]])
    dx = O.avgpool_backward(pooled, (1, 4, 4, 1))
    assert np.array_equal(dx[0, :2, :2, 0], np.full((2, 2), 0.75))
    assert np.array_equal(dx[0, :2, 2:, 0], np.full((2, 2), 1.125))
    assert np.array_equal(dx[0, 2:, :2, 0], np.full((2, 2), 1.875))
    assert np.array_equal(dx[0, 2:, 2:, 0], np.full((2, 2), 1.625))


def test_maxpool_first_max_wins_and_bruteforce():
    x = np.zeros((1, 2, 2, 1), dtype=np.float32)          # all-zero window -> top-left
    _, idx = O.maxpool_forward(x)
    assert idx[0, 0, 0, 0] == 0
    x[0, 0, 1, 0] = x[0, 1, 0, 0] = 3.0                   # tie between flat 1 and 2 -> 1
    _, idx = O.maxpool_forward(x)
    assert idx[0, 0, 0, 0] == 1
    r = np.random.RandomState(0)
    x = r.randint(0, 4, (2, 7, 6, 3)).astype(np.float32)  # many ties, ragged edge
    pooled, idx = O.maxpool_forward(x, (2, 2), (2, 2))
    assert pooled.shape == (2, 3, 3, 3)
    for s in range(2):
        for h in range(3):
            for w in range(3):
                for c in range(3):
                    win = x[s, 2 * h:2 * h + 2, 2 * w:2 * w + 2, c].ravel()
                    best, bi = win[0], 0
                    for k in range(1, 4):
                        if win[k] > best:
                            best, bi = win[k], k
                    assert pooled[s, h, w, c] == best and idx[s, h, w, c] == bi
    dy = r.randn(2, 3, 3, 3).astype(np.float32)
    dx = O.maxpool_backward(dy, idx, x.shape)
    assert np.isclose(dx.sum(), dy.sum(), rtol=1e-5)
    assert np.all(dx[:, 6] == 0)
    # overlapping windows accumulate (np.add.at semantics, nb :155-183)
    x = np.zeros((1, 3, 3, 1), dtype=np.float32)
    x[0, 1, 1, 0] = 5
    pooled, idx = O.maxpool_forward(x, (2, 2), (1, 1))
    dx = O.maxpool_backward(np.ones((1, 2, 2, 1), np.float32), idx, x.shape, (2, 2), (1, 1))
    assert dx[0, 1, 1, 0] == 4


# ---- activations ----------------------------------------------------------------
def test_relu_strictness():
    x = np.array([-1.0, 0.0, 2.0], dtype=np.float32)
    dy = np.array([5.0, 6.0, 7.0], dtype=np.float32)
    assert np.array_equal(O.relu_forward(x), [0, 0, 2])
    assert np.array_equal(O.relu_backward(x, dy), [0, 6, 7])          # passes at x == 0
    assert np.allclose(O.leaky_relu_forward(x, 0.1), [-0.1, 0, 2])
    assert np.allclose(O.leaky_relu_backward(x, dy, 0.1), [0.5, 6, 7])


# ---- batch norm -------------------------------------------------------------------
def test_bn_vs_torch_and_invariants():
    r = np.random.RandomState(1)
    x = r.randn(4, 5, 6, 3) * 2 + 1
    g = r.rand(3) + 0.5
    be = r.randn(3)
    dy = r.randn(4, 5, 6, 3)
    rm, rv = np.zeros(3), np.ones(3)
    y, xhat, mu, var, nrm, nrv = O.bn_forward_train(x, g, be, rm, rv, 1e-5, 0.9)
    xt = torch.from_numpy(x).permute(0, 3, 1, 2).contiguous().requires_grad_(True)
    gt = torch.from_numpy(g).clone().requires_grad_(True)
    bt = torch.from_numpy(be).clone().requires_grad_(True)
    trm, trv = torch.zeros(3, dtype=torch.float64), torch.ones(3, dtype=torch.float64)
    yt = F.batch_norm(xt, trm, trv, gt, bt, training=True, momentum=0.1, eps=1e-5)
    np.testing.assert_allclose(y, yt.detach().permute(0, 2, 3, 1).numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(nrm.ravel(), trm.numpy(), rtol=1e-12)
    # running var: reference keeps the biased variance (torch stores the unbiased one)
    np.testing.assert_allclose(nrv.ravel(), 0.9 + 0.1 * x.var(axis=(0, 1, 2)), rtol=1e-12)
    assert nrm.shape == (1, 1, 1, 3)
    yt.backward(torch.from_numpy(dy).permute(0, 3, 1, 2))
    dx, dg, db = O.bn_backward(x, dy, g, mu, var, 1e-5)
    np.testing.assert_allclose(dx, xt.grad.permute(0, 2, 3, 1).numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=1e-10)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-10)
    assert np.allclose(dx.sum(axis=(0, 1, 2)), 0, atol=1e-10)
    # exact only for eps -> 0: the residual is O(eps / var)
    assert np.allclose((dx * xhat).sum(axis=(0, 1, 2)), 0, atol=1e-4)
    # inference path + 2-D input
    yi = O.bn_forward_infer(x, g, be, nrm, nrv, 1e-5)
    np.testing.assert_allclose(yi, g * (x - nrm) / np.sqrt(nrv + 1e-5) + be, rtol=1e-12)
    x2 = r.randn(8, 3)
    y2, *_ = O.bn_forward_train(x2, np.ones(3), np.zeros(3), rm, rv)
    assert np.allclose(y2.mean(0), 0, atol=1e-12) and np.allclose(y2.var(0), 1, atol=1e-4)


# ---- softmax / loss -----------------------------------------------------------------
def test_softmax_cce_vs_torch():
    r = np.random.RandomState(2)
    logits = r.randn(16, 10) * 3
    y = r.randint(0, 10, 16)
    for ls in (0.0, 0.01, 0.2):
        p = O.softmax(logits)
        loss = O.cce_forward(p, y, ls, training=True)
        lt = torch.from_numpy(logits).clone().requires_grad_(True)
        want = F.cross_entropy(lt, torch.from_numpy(y), label_smoothing=ls, reduction="none")
        np.testing.assert_allclose(loss, want.detach().numpy(), rtol=1e-6, atol=1e-7)
        want.mean().backward()
        np.testing.assert_allclose(O.softmax_cce_backward(p, y, ls), lt.grad.numpy(), rtol=1e-9, atol=1e-12)
    # evaluation ignores smoothing; one-hot labels accepted; clipping bounds the loss
    p = O.softmax(logits)
    np.testing.assert_allclose(O.cce_forward(p, y, 0.2, training=False), O.cce_forward(p, y, 0.0), rtol=0)
    np.testing.assert_allclose(O.cce_forward(p, np.eye(10)[y], 0.0), O.cce_forward(p, y, 0.0), rtol=1e-12)
    hard = np.zeros((1, 10))
    hard[0, 0] = 1.0
    assert np.isclose(O.cce_forward(hard, np.array([1]), 0.0)[0], -np.log(1e-7))


def test_soft_targets_vs_torch():
    """A 2-D y_true is used as given (CNN_classes_cupy.py:622-626, :672-676): rows that are probabilities, not
    one-hot.  torch's cross_entropy takes class probabilities as target and smooths them the same way."""
    r = np.random.RandomState(12)
    logits = r.randn(16, 10) * 1.5                          # (no probability below the reference's clip at 1e-7)
    assert O.softmax(logits).min() > 1e-6
    t = r.rand(16, 10) ** 3
    t /= t.sum(axis=1, keepdims=True)
    for ls in (0.0, 0.05):
        p = O.softmax(logits)
        lt = torch.from_numpy(logits).clone().requires_grad_(True)
        want = F.cross_entropy(lt, torch.from_numpy(t), label_smoothing=ls, reduction="none")
        np.testing.assert_allclose(O.cce_forward(p, t, ls, training=True), want.detach().numpy(), rtol=1e-6, atol=1e-7)
        want.mean().backward()
        np.testing.assert_allclose(O.softmax_cce_backward(p, t, ls), lt.grad.numpy(), rtol=1e-9, atol=1e-12)
    # a dropped smoothing term or targets replaced by their argmax would not pass
    assert not np.allclose(O.cce_forward(p, t, 0.05), O.cce_forward(p, t, 0.0), rtol=1e-3)
    assert not np.allclose(O.cce_forward(p, t, 0.0), O.cce_forward(p, np.argmax(t, axis=1), 0.0), rtol=1e-2)


# ---- Adam ----------------------------------------------------------------------------
def test_adam_vs_torch_and_closed_form():
    r = np.random.RandomState(3)
    th0 = r.randn(50)
    th, m, v = th0.copy(), np.zeros(50), np.zeros(50)
    tt = torch.from_numpy(th0.copy()).requires_grad_(True)
    opt = torch.optim.Adam([tt], lr=1e-3, betas=(0.9, 0.999), eps=1e-7)
    for it in range(5):
        g = r.randn(50)
        th, m, v = O.adam_update(th, g, m, v, 1e-3, it)
        tt.grad = torch.from_numpy(g.copy())
        opt.step()
        np.testing.assert_allclose(th, tt.detach().numpy(), rtol=1e-9, atol=1e-12)
        if it == 0:
            np.testing.assert_allclose(th, th0 - 1e-3 * g / (np.abs(g) + 1e-7), rtol=1e-9)


# ---- the three-block CNN ----------------------------------------------------------------
def test_oracle_cnn_step_matches_torch_autograd():
    """Whole-step check of the chain rule wiring: fp64 oracle vs a torch model
    of the same topology (weights shared), on a tiny batch."""
    np.random.seed(0)
    X = np.random.rand(4, 8, 8, 3)
    y = np.random.randint(0, 10, 4)
    params = O.make_cnn_params(dtype=np.float64, hw=8)
    # larger dense weights so gradients are not vanishingly small
    params[6] = (params[6][0] * 100, params[6][1])
    params[7] = (params[7][0] * 100, params[7][1])
    net = O.OracleCNN(params, label_smoothing=0.01, dtype=np.float64)
    out = net.step(X, y)

    t = lambda a: torch.from_numpy(np.array(a, dtype=np.float64)).requires_grad_(True)
    tp = [[t(a) for a in tup[:2]] for tup in params]
    a = torch.from_numpy(X).permute(0, 3, 1, 2)
    li = 0
    for blk in range(3):
        W, b = tp[li]
        a = F.conv2d(a, W.permute(3, 2, 0, 1), b, padding=1)
        g, be = tp[li + 1]
        a = F.batch_norm(a, None, None, g, be, training=True, eps=1e-5)
        a = F.max_pool2d(F.relu(a), 2)
        li += 2
    a = a.permute(0, 2, 3, 1).reshape(4, -1)
    a = F.leaky_relu(a @ tp[6][0] + tp[6][1], 0.01)
    logits = a @ tp[7][0] + tp[7][1]
    loss = F.cross_entropy(logits, torch.from_numpy(y), label_smoothing=0.01)
    loss.backward()
    assert abs(out["loss"] - loss.item()) < 1e-9
    for i, tup in enumerate(tp):
        for j in range(2):
            got = out["grads"][i][j].reshape(tup[j].shape)
            np.testing.assert_allclose(got, tup[j].grad.numpy(), rtol=1e-6, atol=1e-10)


def test_oracle_cnn_recipe_step_matches_torch_autograd_and_adam():
    """The shipped recipe (CNN/architectures/CNN_cifar1.py:19-55): spatial dropout behind
    the ReLU of blocks 2 and 3, elementwise dropout behind the leaky ReLU, L2 on Dense-1
    and learning-rate decay.  Pinned by a torch graph that the oracle did not write: the
    masks enter as plain multiplications, the L2 penalty as a TERM OF THE LOSS (so autograd
    must produce the 2*lambda*W the oracle adds to dweights by hand, and the penalty value
    must be the oracle's regularization_loss), and the update is torch.optim.Adam stepped
    with the decayed learning rate lr/(1 + decay*t)."""
    np.random.seed(1)
    S = 6
    X = np.random.rand(S, 8, 8, 3)
    y = np.random.randint(0, 10, S)
    params = O.make_cnn_params(dtype=np.float64, hw=8)
    params[6] = (params[6][0] * 100, params[6][1] + 0.3)
    params[7] = (params[7][0] * 100, params[7][1])
    wl2, bl2, decay, lr = 2e-2, 3e-2, 0.5, 1e-3         # large on purpose: a dropped term must show
    net = O.OracleCNN(params, label_smoothing=0.01, lr=lr, decay=decay, dtype=np.float64, dense1_l2=(wl2, bl2))
    r = np.random.RandomState(2)

    t = lambda a: torch.from_numpy(np.array(a, dtype=np.float64)).requires_grad_(True)
    tp = [[t(a) for a in tup[:2]] for tup in params]
    flat = [p for tup in tp for p in tup]
    opt = torch.optim.Adam(flat, lr=lr, betas=(0.9, 0.999), eps=1e-7)
    for step in range(3):
        masks = {"spatial1": r.binomial(1, 0.7, (1, 1, 1, 64)) / 0.7,
                 "spatial2": r.binomial(1, 0.6, (1, 1, 1, 128)) / 0.6,
                 "dense": r.binomial(1, 0.8, (S, 256)) / 0.8}
        out = net.step(X, y, masks=masks)

        a = torch.from_numpy(X).permute(0, 3, 1, 2)
        li = 0
        for blk in range(3):
            W, b = tp[li]
            a = F.conv2d(a, W.permute(3, 2, 0, 1), b, padding=1)
            g, be = tp[li + 1]
            a = F.relu(F.batch_norm(a, None, None, g, be, training=True, eps=1e-5))
            if blk > 0:
                a = a * torch.from_numpy(masks["spatial%d" % blk]).reshape(1, -1, 1, 1)
            a = F.max_pool2d(a, 2)
            li += 2
        a = a.permute(0, 2, 3, 1).reshape(S, -1)
        a = F.leaky_relu(a @ tp[6][0] + tp[6][1], 0.01) * torch.from_numpy(masks["dense"])
        logits = a @ tp[7][0] + tp[7][1]
        data = F.cross_entropy(logits, torch.from_numpy(y), label_smoothing=0.01)
        penalty = wl2 * (tp[6][0] ** 2).sum() + bl2 * (tp[6][1] ** 2).sum()
        opt.zero_grad()
        (data + penalty).backward()
        assert abs(out["loss"] - data.item()) < 1e-9
        assert abs(out["reg_loss"] - penalty.item()) < 1e-12 and out["reg_loss"] > 1e-3
        for i, tup in enumerate(tp):
            for j in range(2):
                got = out["grads"][i][j].reshape(tup[j].shape)
                np.testing.assert_allclose(got, tup[j].grad.numpy(), rtol=1e-6, atol=1e-10)
        want_lr = lr / (1.0 + decay * step)
        assert abs(out["lr"] - want_lr) < 1e-15
        for grp in opt.param_groups:
            grp["lr"] = want_lr
        opt.step()
        for i, tup in enumerate(tp):
            for j in range(2):
                np.testing.assert_allclose(net.p[i][j], tup[j].detach().numpy().reshape(net.p[i][j].shape),
                                           rtol=1e-7, atol=1e-10)
    # evaluation ignores the masks
    p_eval, _ = net.forward(X, training=False, masks=masks)
    p_eval2, _ = net.forward(X, training=False)
    assert np.array_equal(p_eval, p_eval2)
