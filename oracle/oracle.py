"""NumPy restatement of the reference's convolution hot path and of the layers
either side of it.  TEST INFRASTRUCTURE ONLY -- the product never imports this.

Every function cites the reference lines it follows (paths are relative to the
reference checkout; ``classes`` = CNN/models/CNN_classes.py, ``cupy`` =
CNN/models/CNN_classes_cupy.py).  The arithmetic is the reference's own
``as_strided`` + ``einsum`` formulation with two stated departures:

* ``conv_dgrad`` accumulates every tap (what the CuPy scatter kernel does with
  atomicAdd, cupy:4-35,138-146).  The NumPy file's ``dinput_patches +=
  contributions`` (classes:102-116) writes through an overlapping view and
  keeps only the last-written tap; that behaviour is reproduced by
  ``numpy_reference_quirk=True`` purely so tests can show it is not a gradient.
* ``conv_dgrad`` with P == 0 returns the full tensor (the reference's
  ``[:, P:-P, P:-P, :]`` slice is empty when P == 0 under "same",
  classes:119-121).

What pins each function (see tests/test_oracle_*.py):
  conv_fprop  -- notebook known answers, 7-loop brute force, torch conv2d
  conv_wgrad  -- torch autograd, finite differences, <dW,W> = <dy,y-b>
  conv_dbias  -- closed form
  conv_dgrad  -- notebook worked example, torch autograd, adjoint identity
  dense_*     -- fp64 matmul, torch linear
  maxpool     -- notebook 4x4 example, brute force, first-max tie rule
  batch norm  -- torch batch_norm + invariants
  softmax/CCE -- torch cross_entropy(label_smoothing)
  adam        -- torch.optim.Adam(eps=1e-7), step-1 closed form
  dropout, regularization_loss, learning-rate decay, the L2 terms of dense_backward
              -- three steps of OracleCNN with masks, L2 and decay against a torch
                 graph (masks as multiplications, the penalty as a term of the loss,
                 torch.optim.Adam stepped at lr/(1+decay*t))
"""
from __future__ import annotations

import numpy as np
from numpy.lib.stride_tricks import as_strided


# ----------------------------------------------------------------------------
# geometry
# ----------------------------------------------------------------------------
def conv_geometry(H, W, fH, fW, sH, sW, padding):
    """P, Ho, Wo exactly as classes:40-47 / cupy:78-85.

    P comes from fH only, is applied to both axes and ignores the stride.
    """
    if padding == "same":
        P = (fH - 1) // 2
    else:
        P = 0
    Ho = int((H + 2 * P - fH) / sH + 1)
    Wo = int((W + 2 * P - fW) / sW + 1)
    return P, Ho, Wo


def _patches(xpad, Ho, Wo, fH, fW, sH, sW):
    """6-D sliding-window view [S,Ho,Wo,fH,fW,C] (classes:63-74)."""
    S, _, _, C = xpad.shape
    st = xpad.strides
    return as_strided(
        xpad,
        shape=(S, Ho, Wo, fH, fW, C),
        strides=(st[0], st[1] * sH, st[2] * sW, st[1], st[2], st[3]),
        writeable=False,
    )


def _pad(x, P):
    """Zero pad H and W by P (classes:54-57)."""
    return np.pad(x, ((0, 0), (P, P), (P, P), (0, 0)), mode="constant", constant_values=0)


# ----------------------------------------------------------------------------
# convolution
# ----------------------------------------------------------------------------
def conv_fprop(x, w, b, strides=(1, 1), padding="same", dtype=np.float32):
    """y[s,h,w,d] = b[d] + sum_{x,y,c} xpad[s,h*sH+x,w*sW+y,c] * W[x,y,c,d].

    classes:32-82 (einsum at :77, bias add at :78); cupy:70-120.
    """
    x = np.asarray(x, dtype=dtype)
    w = np.asarray(w, dtype=dtype)
    fH, fW, C, D = w.shape
    sH, sW = strides
    S, H, W_, Cx = x.shape
    assert Cx == C
    P, Ho, Wo = conv_geometry(H, W_, fH, fW, sH, sW, padding)
    xpad = _pad(x, P)
    pat = _patches(xpad, Ho, Wo, fH, fW, sH, sW)
    y = np.einsum("shwxyc,xycd->shwd", pat, w)
    if b is not None:
        y = y + np.asarray(b, dtype=dtype).reshape(1, 1, 1, D)
    return y.astype(dtype, copy=False)


def conv_dbias(dy, dtype=np.float32):
    """db[d] = sum_{s,h,w} dy[s,h,w,d]  (classes:92, cupy:132)."""
    return np.sum(np.asarray(dy, dtype=dtype), axis=(0, 1, 2))


def conv_wgrad(x, dy, filter_size, strides=(1, 1), padding="same", dtype=np.float32):
    """dW[x,y,c,d] = sum_{s,h,w} xpad[s,h*sH+x,w*sW+y,c] * dy[s,h,w,d].

    classes:94, cupy:134.
    """
    x = np.asarray(x, dtype=dtype)
    dy = np.asarray(dy, dtype=dtype)
    fH, fW = filter_size
    sH, sW = strides
    S, H, W_, C = x.shape
    P, Ho, Wo = conv_geometry(H, W_, fH, fW, sH, sW, padding)
    assert dy.shape[:3] == (S, Ho, Wo)
    pat = _patches(_pad(x, P), Ho, Wo, fH, fW, sH, sW)
    return np.einsum("shwxyc,shwd->xycd", pat, dy).astype(dtype, copy=False)


def conv_dgrad(dy, w, input_hw, strides=(1, 1), padding="same", dtype=np.float32,
               numpy_reference_quirk=False):
    """dx[s,i,j,c] = sum over taps (h*sH+x = i+P, w*sW+y = j+P) and d of
    dy[s,h,w,d] * W[x,y,c,d]; the padded border is cropped.

    contributions = einsum("shwd,xycd->shwxyc") (classes:98, cupy:138) followed
    by a scatter into the padded gradient.  The scatter here accumulates
    (cupy:24-32).  With ``numpy_reference_quirk`` the last write in C order of
    (s,h,w,x,y,c) wins instead, which is what classes:116 does.
    """
    dy = np.asarray(dy, dtype=dtype)
    w = np.asarray(w, dtype=dtype)
    fH, fW, C, D = w.shape
    sH, sW = strides
    H, W_ = input_hw
    S, Ho, Wo, Dy = dy.shape
    assert Dy == D
    P, Ho2, Wo2 = conv_geometry(H, W_, fH, fW, sH, sW, padding)
    assert (Ho, Wo) == (Ho2, Wo2)
    contrib = np.einsum("shwd,xycd->shwxyc", dy, w)
    dxpad = np.zeros((S, H + 2 * P, W_ + 2 * P, C), dtype=dtype)
    if numpy_reference_quirk:
        # A padded pixel is covered by at most one (x,y) of a given window, so
        # assigning whole windows in (h,w) order leaves the C-order last writer.
        for h in range(Ho):
            for w_ in range(Wo):
                dxpad[:, h * sH:h * sH + fH, w_ * sW:w_ * sW + fW, :] = contrib[:, h, w_]
    else:
        for fx in range(fH):
            for fy in range(fW):
                dxpad[:, fx:fx + (Ho - 1) * sH + 1:sH, fy:fy + (Wo - 1) * sW + 1:sW, :] += \
                    contrib[:, :, :, fx, fy, :]
    if P > 0:
        return dxpad[:, P:-P, P:-P, :]
    return dxpad


def conv_fprop_bruteforce(x, w, b, strides, padding):
    """Seven nested loops in float64; for tiny shapes only."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    fH, fW, C, D = w.shape
    sH, sW = strides
    S, H, W_, _ = x.shape
    P, Ho, Wo = conv_geometry(H, W_, fH, fW, sH, sW, padding)
    y = np.zeros((S, Ho, Wo, D))
    for s in range(S):
        for h in range(Ho):
            for ww in range(Wo):
                for d in range(D):
                    acc = 0.0 if b is None else float(b[d])
                    for fx in range(fH):
                        for fy in range(fW):
                            i = h * sH + fx - P
                            j = ww * sW + fy - P
                            if 0 <= i < H and 0 <= j < W_:
                                for c in range(C):
                                    acc += x[s, i, j, c] * w[fx, fy, c, d]
                    y[s, h, ww, d] = acc
    return y


def conv_dgrad_bruteforce(dy, w, input_hw, strides, padding):
    """Scatter form in float64 (the CuPy kernel's loop, cupy:14-32)."""
    dy = np.asarray(dy, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    fH, fW, C, D = w.shape
    sH, sW = strides
    H, W_ = input_hw
    S, Ho, Wo, _ = dy.shape
    P, _, _ = conv_geometry(H, W_, fH, fW, sH, sW, padding)
    dxp = np.zeros((S, H + 2 * P, W_ + 2 * P, C))
    for s in range(S):
        for h in range(Ho):
            for ww in range(Wo):
                for fx in range(fH):
                    for fy in range(fW):
                        for c in range(C):
                            dxp[s, h * sH + fx, ww * sW + fy, c] += float(
                                np.dot(dy[s, h, ww, :], w[fx, fy, c, :]))
    return dxp[:, P:P + H, P:P + W_, :]


# ----------------------------------------------------------------------------
# dense
# ----------------------------------------------------------------------------
def dense_forward(x, w, b, dtype=np.float32):
    """Y = X.W + b (classes:255-259, cupy:328-331)."""
    x = np.asarray(x, dtype=dtype)
    return (np.dot(x, np.asarray(w, dtype=dtype)) + np.asarray(b, dtype=dtype)).astype(dtype, copy=False)


def dense_backward(x, w, b, dy, wl1=0.0, wl2=0.0, bl1=0.0, bl2=0.0, dtype=np.float32):
    """dW = X^T.dY (+reg), db = sum_s dY (+reg), dX = dY.W^T (classes:261-284).

    L1 uses sign(0) = +1 (classes:265-267).
    """
    x = np.asarray(x, dtype=dtype)
    w = np.asarray(w, dtype=dtype)
    b = np.asarray(b, dtype=dtype)
    dy = np.asarray(dy, dtype=dtype)
    dw = np.dot(x.T, dy)
    db = np.sum(dy, axis=0, keepdims=True)
    if wl1 > 0:
        dl1 = np.ones_like(w)
        dl1[w < 0] = -1
        dw = dw + dtype(wl1) * dl1
    if wl2 > 0:
        dw = dw + dtype(2 * wl2) * w
    if bl1 > 0:
        dl1 = np.ones_like(b)
        dl1[b < 0] = -1
        db = db + dtype(bl1) * dl1
    if bl2 > 0:
        db = db + dtype(2 * bl2) * b
    dx = np.dot(dy, w.T)
    return dw.astype(dtype, copy=False), db.astype(dtype, copy=False), dx.astype(dtype, copy=False)


# ----------------------------------------------------------------------------
# activations
# ----------------------------------------------------------------------------
def relu_forward(x):
    """max(0, x) (cupy:408-411)."""
    return np.maximum(0, x)


def relu_backward(x, dy):
    """dx = dy, zero where x < 0 -- strict (cupy:413-415)."""
    dx = np.array(dy, copy=True)
    dx[x < 0] = 0
    return dx


def leaky_relu_forward(x, alpha=0.01):
    """where(x > 0, x, alpha*x) (cupy:421-424)."""
    return np.where(x > 0, x, x.dtype.type(alpha) * x)


def leaky_relu_backward(x, dy, alpha=0.01):
    """dx = dy, scaled by alpha where x < 0 (cupy:426-428)."""
    dx = np.array(dy, copy=True)
    dx[x < 0] *= dx.dtype.type(alpha)
    return dx


# ----------------------------------------------------------------------------
# max pooling ("valid" only; "same" is broken upstream, cupy:226-228)
# ----------------------------------------------------------------------------
def maxpool_forward(x, filter_size=(2, 2), strides=(2, 2), dtype=np.float32):
    """Window max and flat argmax (first maximum in row-major window order),
    cupy:212-273.  Returns (pooled, flat_index[int]).  The reference casts the
    input to float32 (cupy:214); ``dtype`` lets a float64 evaluation opt out."""
    x = np.asarray(x, dtype=dtype)
    S, H, W_, C = x.shape
    fH, fW = filter_size
    sH, sW = strides
    Ho = int(np.floor((H - fH) / sH + 1))
    Wo = int(np.floor((W_ - fW) / sW + 1))
    st = x.strides
    pat = as_strided(x, shape=(S, Ho, Wo, fH, fW, C),
                     strides=(st[0], st[1] * sH, st[2] * sW, st[1], st[2], st[3]),
                     writeable=False)
    pooled = pat.max(axis=(3, 4))
    flat = pat.reshape(S, Ho, Wo, fH * fW, C).argmax(axis=3)
    return pooled, flat


def maxpool_backward(dy, flat_idx, input_shape, filter_size=(2, 2), strides=(2, 2), dtype=np.float32):
    """Scatter-add of dy at the argmax positions (cupy:275-300)."""
    dy = np.asarray(dy, dtype=dtype)
    S, Ho, Wo, C = dy.shape
    fH, fW = filter_size
    sH, sW = strides
    rows, cols = np.unravel_index(flat_idx, (fH, fW))
    dx = np.zeros(input_shape, dtype=dtype)
    s_idx = np.arange(S)[:, None, None, None]
    h_idx = np.arange(Ho)[None, :, None, None]
    w_idx = np.arange(Wo)[None, None, :, None]
    c_idx = np.arange(C)[None, None, None, :]
    np.add.at(dx, (s_idx, h_idx * sH + rows, w_idx * sW + cols, c_idx), dy)
    return dx


def avgpool_forward(x, filter_size=(2, 2), strides=(2, 2)):
    """Window mean (cupy:267-268)."""
    x = np.asarray(x, dtype=np.float32)
    S, H, W_, C = x.shape
    fH, fW = filter_size
    sH, sW = strides
    Ho = int(np.floor((H - fH) / sH + 1))
    Wo = int(np.floor((W_ - fW) / sW + 1))
    st = x.strides
    pat = as_strided(x, shape=(S, Ho, Wo, fH, fW, C),
                     strides=(st[0], st[1] * sH, st[2] * sW, st[1], st[2], st[3]),
                     writeable=False)
    return pat.mean(axis=(3, 4))


def avgpool_backward(dy, input_shape, filter_size=(2, 2), strides=(2, 2)):
    """Each window position receives dy/(fH*fW), accumulating over overlapping
    windows (scatter kernel cupy:163-202)."""
    dy = np.asarray(dy, dtype=np.float32)
    S, Ho, Wo, C = dy.shape
    fH, fW = filter_size
    sH, sW = strides
    dx = np.zeros(input_shape, dtype=np.float32)
    g = dy / np.float32(fH * fW)
    for fx in range(fH):
        for fy in range(fW):
            dx[:, fx:fx + (Ho - 1) * sH + 1:sH, fy:fy + (Wo - 1) * sW + 1:sW, :] += g
    return dx


# ----------------------------------------------------------------------------
# batch norm
# ----------------------------------------------------------------------------
def _bn_axes(x):
    return (0, 1, 2) if x.ndim == 4 else (0,)


def bn_forward_train(x, gamma, beta, running_mean, running_var, eps=1e-5, momentum=0.9):
    """cupy:467-476.  Returns (y, xhat, batch_mean, batch_var, new_rm, new_rv);
    variance is the biased one, running stats keep the keepdims shape."""
    axes = _bn_axes(x)
    mu = np.mean(x, axis=axes, keepdims=True)
    var = np.var(x, axis=axes, keepdims=True)
    xhat = (x - mu) / np.sqrt(var + x.dtype.type(eps))
    y = gamma * xhat + beta
    m = x.dtype.type(momentum)
    one_m = x.dtype.type(1 - momentum)
    rm = m * running_mean + one_m * mu
    rv = m * running_var + one_m * var
    return y, xhat, mu, var, rm, rv


def bn_forward_infer(x, gamma, beta, running_mean, running_var, eps=1e-5):
    """cupy:478-480."""
    xhat = (x - running_mean) / np.sqrt(running_var + x.dtype.type(eps))
    return gamma * xhat + beta


def bn_backward(x, dy, gamma, mu, var, eps=1e-5):
    """cupy:484-508.  Returns (dx, dgamma, dbeta)."""
    axes = _bn_axes(dy)
    dt = x.dtype.type
    N = dt(np.prod([x.shape[a] for a in axes]))
    dhat = dy * gamma
    xc = x - mu
    dvar = np.sum(dhat * xc * dt(-0.5) * np.power(var + dt(eps), dt(-1.5)), axis=axes, keepdims=True)
    inv = dt(1.0) / np.sqrt(var + dt(eps))
    dmu = np.sum(dhat * (-inv), axis=axes, keepdims=True) + \
        dvar * np.sum(dt(-2.0) * xc, axis=axes, keepdims=True) / N
    dx = dhat * inv + dvar * dt(2.0) * xc / N + dmu / N
    xhat = xc * inv
    dgamma = np.sum(dy * xhat, axis=axes)
    dbeta = np.sum(dy, axis=axes)
    return dx, dgamma, dbeta


# ----------------------------------------------------------------------------
# softmax / loss
# ----------------------------------------------------------------------------
def softmax(x):
    """cupy:542-547."""
    e = np.exp(x - np.max(x, axis=1, keepdims=True))
    return e / np.sum(e, axis=1, keepdims=True)


def _smooth_targets(y_true, n_classes, label_smoothing, dtype):
    if y_true.ndim == 1:
        t = np.eye(n_classes, dtype=dtype)[y_true]
    else:
        t = np.asarray(y_true, dtype=dtype)
    if label_smoothing > 0:
        t = t * dtype(1.0 - label_smoothing) + dtype(label_smoothing / n_classes)
    return t


def cce_forward(probs, y_true, label_smoothing=0.0, training=True):
    """Per-sample loss, clip to [1e-7, 1-1e-7], smoothing only when training
    (cupy:615-632)."""
    K = probs.shape[1]
    dt = probs.dtype.type
    p = np.clip(probs, dt(1e-7), dt(1 - 1e-7))
    t = _smooth_targets(y_true, K, label_smoothing if training else 0.0, dt)
    return -np.sum(t * np.log(p), axis=1)


def softmax_cce_backward(probs, y_true, label_smoothing=0.0):
    """(p - t_smooth) / S with the unclipped p (cupy:666-680)."""
    S, K = probs.shape
    t = _smooth_targets(y_true, K, label_smoothing, probs.dtype.type)
    return (probs - t) / probs.dtype.type(S)


# ----------------------------------------------------------------------------
# Adam
# ----------------------------------------------------------------------------
def adam_update(theta, g, m, v, lr, iterations, beta1=0.9, beta2=0.999, eps=1e-7):
    """One tensor's update, cupy:702-734.  ``iterations`` is the 0-based count
    before this step.  Returns (theta, m, v)."""
    dt = theta.dtype.type
    m = dt(beta1) * m + dt(1 - beta1) * g
    v = dt(beta2) * v + dt(1 - beta2) * (g * g)
    mhat = m / dt(1 - beta1 ** (iterations + 1))
    vhat = v / dt(1 - beta2 ** (iterations + 1))
    theta = theta + (-dt(lr)) * mhat / (np.sqrt(vhat) + dt(eps))
    return theta, m, v


# ----------------------------------------------------------------------------
# bf16 helpers
# ----------------------------------------------------------------------------
def round_to_bf16(a):
    """fp32 -> bf16 (round to nearest even) -> fp32, as a float32 array."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    nan = np.isnan(a)
    out = rounded.astype(np.uint32).view(np.float32)
    if nan.any():
        out = out.copy()
        out[nan] = np.nan
    return out.reshape(a.shape)


def bf16_bits(a):
    """fp32 array -> uint16 array of bf16 bit patterns (RNE)."""
    return (round_to_bf16(a).view(np.uint32) >> 16).astype(np.uint16)


# ----------------------------------------------------------------------------
# dropout and the regulariser term of the loss
# ----------------------------------------------------------------------------
def dropout_forward(x, mask):
    """Layer_Dropout / Layer_Dropout_Spatial in training (cupy:375-377, :396-399):
    output = inputs * mask, where the mask already holds Bernoulli(keep)/keep.
    Elementwise dropout passes a mask of the input's shape, spatial dropout one of
    shape (1,1,1,C) that every sample and pixel shares."""
    return x * np.asarray(mask, dtype=x.dtype)


def dropout_backward(dy, mask):
    """dinputs = dvalues * mask (cupy:381-382, :402-403)."""
    return dy * np.asarray(mask, dtype=dy.dtype)


def regularization_loss(weights, biases, wl1=0.0, wl2=0.0, bl1=0.0, bl2=0.0):
    """One layer's share of Loss.regularization_loss (cupy:593-609):
    l1*sum|w| + l2*sum w^2 for weights and biases, each term only when its
    coefficient is positive."""
    w = np.asarray(weights)
    b = np.asarray(biases)
    r = 0.0
    if wl1 > 0:
        r += wl1 * np.sum(np.abs(w))
    if wl2 > 0:
        r += wl2 * np.sum(w * w)
    if bl1 > 0:
        r += bl1 * np.sum(np.abs(b))
    if bl2 > 0:
        r += bl2 * np.sum(b * b)
    return float(r)


# ----------------------------------------------------------------------------
# The three-block CNN of the headline training step, as a plain function chain
# (topology: CNN/architectures/CNN_cifar1.py:19-47; the dropout layers and the
# regulariser of that script are optional)
# ----------------------------------------------------------------------------
class OracleCNN:
    """Conv(32)-BN-ReLU-Pool, Conv(64)-BN-ReLU-[SpatialDropout]-Pool,
    Conv(128)-BN-ReLU-[SpatialDropout]-Pool, Flatten, Dense(256) LeakyReLU(0.01)
    [Dropout], Dense(10), softmax CCE, Adam.

    ``params`` is the list of per-layer tuples in trainable-layer order
    (conv W,b / bn gamma,beta,rm,rv / dense W,b), all float arrays of
    ``dtype``.  ``step`` performs forward, loss, backward and the Adam update
    and returns a dict of every intermediate a parity test wants.

    The shipped recipe (CNN_cifar1.py:30,38,43,45,51) adds spatial dropout behind
    the ReLU of blocks 2 and 3, elementwise dropout behind the leaky ReLU, an L2
    penalty on Dense-1's weights and biases and learning-rate decay.  Masks are
    passed per step as ``masks={"spatial1": (1,1,1,64), "spatial2": (1,1,1,128),
    "dense": (S,256)}`` (values Bernoulli(keep)/keep, any of them optional); the
    L2 coefficients as ``dense1_l2=(weight_l2, bias_l2)``.
    """

    def __init__(self, params, label_smoothing=0.01, lr=1e-3, decay=0.0, dtype=np.float32,
                 eps_bn=1e-5, momentum=0.9, dense1_l2=(0.0, 0.0)):
        self.dt = dtype
        self.p = [[np.array(a, dtype=dtype) for a in tup] for tup in params]
        self.ls = label_smoothing
        self.lr = lr
        self.decay = decay
        self.iterations = 0
        self.current_lr = lr
        self.eps_bn = eps_bn
        self.momentum = momentum
        self.dense1_l2 = tuple(dense1_l2)
        self.m = [[np.zeros_like(a) for a in tup[:2]] for tup in self.p]
        self.v = [[np.zeros_like(a) for a in tup[:2]] for tup in self.p]

    def regularization_loss(self):
        """Loss.regularization_loss over the trainable layers (cupy:593-609): only
        Dense-1 carries coefficients in this network."""
        W, b = self.p[6]
        return regularization_loss(W, b, wl2=self.dense1_l2[0], bl2=self.dense1_l2[1])

    def forward(self, X, training=True, masks=None):
        dt = self.dt
        masks = masks or {}
        a = np.asarray(X, dtype=dt)
        cache = {}
        li = 0
        for blk in range(3):
            W, b = self.p[li]
            cache[f"conv{blk}_in"] = a
            a = conv_fprop(a, W, b, (1, 1), "same", dtype=dt)
            cache[f"conv{blk}_out"] = a
            g, be, rm, rv = self.p[li + 1]
            if training:
                y, xhat, mu, var, nrm, nrv = bn_forward_train(a, g, be, rm, rv, self.eps_bn, self.momentum)
                cache[f"bn{blk}"] = (a, mu, var)
                self.p[li + 1][2] = nrm.astype(dt)
                self.p[li + 1][3] = nrv.astype(dt)
                a = y.astype(dt)
            else:
                a = bn_forward_infer(a, g, be, rm, rv, self.eps_bn).astype(dt)
            cache[f"bn{blk}_out"] = a
            cache[f"relu{blk}_in"] = a
            a = relu_forward(a)
            mask = masks.get(f"spatial{blk}") if training else None
            cache[f"spatial{blk}"] = mask
            if mask is not None:
                a = dropout_forward(a, np.asarray(mask).reshape(1, 1, 1, -1)).astype(dt)
            pooled, idx = maxpool_forward(a, dtype=dt)
            cache[f"pool{blk}"] = (idx, a.shape)
            a = pooled.astype(dt)
            cache[f"pool{blk}_out"] = a
            li += 2
        cache["flat_shape"] = a.shape
        a = a.reshape(a.shape[0], -1)
        W, b = self.p[li]
        cache["d0_in"] = a
        a = dense_forward(a, W, b, dtype=dt)
        cache["leaky_in"] = a
        a = leaky_relu_forward(a, 0.01).astype(dt)
        mask = masks.get("dense") if training else None
        cache["dense_mask"] = mask
        if mask is not None:
            a = dropout_forward(a, mask).astype(dt)
        W, b = self.p[li + 1]
        cache["d1_in"] = a
        a = dense_forward(a, W, b, dtype=dt)
        cache["logits"] = a
        probs = softmax(a).astype(dt)
        cache["probs"] = probs
        return probs, cache

    def step(self, X, y, masks=None):
        dt = self.dt
        probs, c = self.forward(X, training=True, masks=masks)
        losses = cce_forward(probs, y, self.ls, training=True)
        loss = float(np.mean(losses))
        reg_loss = self.regularization_loss()            # with the parameters before the update (model_cupy:113-115)
        acc = float(np.mean(np.argmax(probs, axis=1) == y))
        grads = [None] * len(self.p)
        d = softmax_cce_backward(probs, y, self.ls).astype(dt)
        c["dlogits"] = d
        li = len(self.p) - 1
        W, b = self.p[li]
        dw, db, d = dense_backward(c["d1_in"], W, b, d, dtype=dt)
        grads[li] = (dw, db)
        if c["dense_mask"] is not None:
            d = dropout_backward(d, c["dense_mask"]).astype(dt)
        d = leaky_relu_backward(c["leaky_in"], d, 0.01)
        li -= 1
        W, b = self.p[li]
        dw, db, d = dense_backward(c["d0_in"], W, b, d, wl2=self.dense1_l2[0], bl2=self.dense1_l2[1], dtype=dt)
        grads[li] = (dw, db)
        d = d.reshape(c["flat_shape"])
        dinputs = {}
        for blk in (2, 1, 0):
            idx, shp = c[f"pool{blk}"]
            d = maxpool_backward(d, idx, shp, dtype=dt)
            if c[f"spatial{blk}"] is not None:
                d = dropout_backward(d, np.asarray(c[f"spatial{blk}"]).reshape(1, 1, 1, -1)).astype(dt)
            d = relu_backward(c[f"relu{blk}_in"], d)
            li -= 1
            g = self.p[li][0]
            xin, mu, var = c[f"bn{blk}"]
            d, dg, dbeta = bn_backward(xin, d, g, mu, var, self.eps_bn)
            d = d.astype(dt)
            grads[li] = (dg.astype(dt), dbeta.astype(dt))
            li -= 1
            W, b = self.p[li]
            xin = c[f"conv{blk}_in"]
            grads[li] = (conv_wgrad(xin, d, W.shape[:2], (1, 1), "same", dtype=dt), conv_dbias(d, dtype=dt))
            d = conv_dgrad(d, W, xin.shape[1:3], (1, 1), "same", dtype=dt)
            dinputs[f"conv{blk}"] = d
        lr = self.lr
        if self.decay:
            lr = self.lr * (1.0 / (1.0 + self.decay * self.iterations))      # pre_update_parameters, cupy:695-697
        self.current_lr = lr
        for i, tup in enumerate(self.p):
            for j in range(2):
                gj = grads[i][j].reshape(tup[j].shape)
                th, m, v = adam_update(tup[j], gj, self.m[i][j], self.v[i][j], lr, self.iterations)
                self.p[i][j] = th.astype(dt)
                self.m[i][j] = m.astype(dt)
                self.v[i][j] = v.astype(dt)
        self.iterations += 1
        return {"loss": loss, "reg_loss": reg_loss, "acc": acc, "probs": probs, "grads": grads, "dinputs": dinputs,
                "cache": c, "lr": lr}


def make_cnn_params(rng_module=np.random, dtype=np.float32, in_ch=3, hw=32):
    """Parameter tuples of the three-block CNN drawn in model order from the
    legacy global RNG, with the reference's initialisers (cupy:54-66 conv
    He-normal; cupy:320-322 dense 0.01*randn*sqrt(2/n_in); BN ones/zeros with
    running mean 0 / var 1, cupy:455-458)."""
    params = []
    c = in_ch
    for d in (32, 64, 128):
        w = (rng_module.randn(3, 3, c, d) * np.sqrt(2.0 / (9 * c))).astype(dtype)
        params.append((w, np.zeros(d, dtype=dtype)))
        params.append((np.ones(d, dtype=dtype), np.zeros(d, dtype=dtype),
                       np.zeros(d, dtype=dtype), np.ones(d, dtype=dtype)))
        c = d
    hw_out = hw // 8
    n_in = hw_out * hw_out * 128
    params.append(((0.01 * rng_module.randn(n_in, 256) * np.sqrt(2.0 / n_in)).astype(dtype),
                   np.zeros((1, 256), dtype=dtype)))
    params.append(((0.01 * rng_module.randn(256, 10) * np.sqrt(2.0 / 256)).astype(dtype),
                   np.zeros((1, 10), dtype=dtype)))
    return params
