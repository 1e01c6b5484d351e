"""Pins the convolution / dense part of the CPU oracle against things it did
not write itself: the reference notebooks' known answers, brute-force loops,
torch's CPU conv2d + autograd, finite differences and adjoint identities."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O

CASES = [
    # S, H, W, C, D, fH, fW, sH, sW, padding
    (2, 5, 5, 1, 1, 3, 3, 1, 1, "valid"),
    (2, 6, 7, 3, 4, 3, 3, 1, 1, "same"),
    (3, 8, 8, 4, 5, 3, 3, 2, 2, "valid"),
    (2, 9, 7, 2, 3, 3, 3, 2, 2, "same"),
    (2, 7, 7, 4, 6, 1, 1, 1, 1, "valid"),
    (1, 8, 9, 3, 2, 5, 3, 1, 2, "same"),
    (2, 6, 6, 2, 2, 2, 2, 2, 2, "valid"),
    (1, 10, 10, 2, 3, 3, 3, 3, 3, "valid"),
]


def _rand_case(case, seed=0, dtype=np.float64):
    S, H, W, C, D, fH, fW, sH, sW, pad = case
    r = np.random.RandomState(seed)
    x = r.randn(S, H, W, C).astype(dtype)
    w = r.randn(fH, fW, C, D).astype(dtype)
    b = r.randn(D).astype(dtype)
    P, Ho, Wo = O.conv_geometry(H, W, fH, fW, sH, sW, pad)
    dy = r.randn(S, Ho, Wo, D).astype(dtype)
    return x, w, b, dy, P


def _torch_conv(x, w, b, stride, P):
    xt = torch.from_numpy(x).permute(0, 3, 1, 2).contiguous().requires_grad_(True)
    wt = torch.from_numpy(w).permute(3, 2, 0, 1).contiguous().requires_grad_(True)
    bt = torch.from_numpy(b).clone().requires_grad_(True)
    y = F.conv2d(xt, wt, bt, stride=stride, padding=P)
    return xt, wt, bt, y


# ---- known answers held by the reference notebooks --------------------------
def test_notebook_edge_kernel_4x4():
    # CNN/notebooks/CNN_Implementation.ipynb:421-472 -> output :411-414
    img = np.array([[1, 2, 3, 0], [0, 1, 2, 3], [3, 0, 1, 2], [2, 3, 0, 1]], dtype=np.float64)
    k = np.array([[1, 0, -1]] * 3, dtype=np.float64)
    y = O.conv_fprop(img[None, :, :, None], k[:, :, None, None], None, (1, 1), "same", dtype=np.float64)
    want = np.array([[-3, -4, 0, 5], [-3, -2, -2, 6], [-4, 2, -2, 3], [-3, 4, 0, 1]], dtype=np.float64)
    assert np.array_equal(y[0, :, :, 0], want)


def test_notebook_ones_valid_9_27_18():
    # CNN_Implementation.ipynb:747-752 (9), :774-779 (27), :803-811 (9 and 18)
    y = O.conv_fprop(np.ones((1, 5, 5, 1)), np.ones((3, 3, 1, 1)), np.zeros(1), (1, 1), "valid")
    assert y.shape == (1, 3, 3, 1) and np.all(y == 9)
    y = O.conv_fprop(np.ones((1, 5, 5, 3)), np.ones((3, 3, 3, 1)), np.zeros(1), (1, 1), "valid")
    assert np.all(y == 27)
    w = np.ones((3, 3, 1, 2))
    w[..., 1] = 2
    y = O.conv_fprop(np.ones((1, 5, 5, 1)), w, np.zeros(2), (1, 1), "valid")
    assert np.all(y[..., 0] == 9) and np.all(y[..., 1] == 18)


def test_notebook_dgrad_worked_example_accumulates():
    # CNN/notebooks/Backpropagation_Conv.ipynb:84-110: ones 3x3 filter, dvalues
    # row "1 2 3 0": after two taps the padded row reads 1 3 3 2 0 0.
    dy = np.zeros((1, 4, 4, 1))
    dy[0, 0, :, 0] = [1, 2, 3, 0]
    w = np.ones((3, 3, 1, 1))
    dx = O.conv_dgrad(dy, w, (4, 4), (1, 1), "same", dtype=np.float64)
    # full accumulation along the first padded row: [1,3,6,5,3,0] -> cropped [3,6,5,3]
    assert np.array_equal(dx[0, 0, :, 0], [3, 6, 5, 3])
    # the first two taps alone give 1 3 3 2 0 0 as the notebook writes
    part = np.zeros(6)
    part[0:3] += 1
    part[1:4] += 2
    assert np.array_equal(part, [1, 3, 3, 2, 0, 0])


# ---- geometry -----------------------------------------------------------------
def test_geometry_rules():
    assert O.conv_geometry(32, 32, 3, 3, 1, 1, "same") == (1, 32, 32)
    assert O.conv_geometry(28, 28, 3, 3, 2, 2, "valid") == (0, 13, 13)
    assert O.conv_geometry(56, 56, 1, 1, 1, 1, "same") == (0, 56, 56)
    # P from fH only, applied to both axes, stride ignored
    assert O.conv_geometry(8, 9, 5, 3, 1, 2, "same") == (2, 8, 6)


# ---- brute force / torch ------------------------------------------------------
@pytest.mark.parametrize("case", CASES)
def test_fprop_vs_bruteforce_and_torch(case):
    x, w, b, dy, P = _rand_case(case)
    stride = (case[7], case[8])
    y = O.conv_fprop(x, w, b, stride, case[9], dtype=np.float64)
    yb = O.conv_fprop_bruteforce(x, w, b, stride, case[9])
    np.testing.assert_allclose(y, yb, rtol=1e-12, atol=1e-12)
    _, _, _, yt = _torch_conv(x, w, b, stride, P)
    np.testing.assert_allclose(y, yt.detach().permute(0, 2, 3, 1).numpy(), rtol=1e-11, atol=1e-11)


@pytest.mark.parametrize("case", CASES)
def test_backward_vs_torch_autograd(case):
    x, w, b, dy, P = _rand_case(case, seed=1)
    stride = (case[7], case[8])
    xt, wt, bt, yt = _torch_conv(x, w, b, stride, P)
    yt.backward(torch.from_numpy(dy).permute(0, 3, 1, 2))
    dw = O.conv_wgrad(x, dy, w.shape[:2], stride, case[9], dtype=np.float64)
    db = O.conv_dbias(dy, dtype=np.float64)
    dx = O.conv_dgrad(dy, w, x.shape[1:3], stride, case[9], dtype=np.float64)
    np.testing.assert_allclose(dw, wt.grad.permute(2, 3, 1, 0).numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-10, atol=1e-10)
    assert dx.shape == x.shape
    np.testing.assert_allclose(dx, xt.grad.permute(0, 2, 3, 1).numpy(), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("case", CASES[:5])
def test_dgrad_vs_scatter_bruteforce(case):
    x, w, b, dy, P = _rand_case(case, seed=2)
    stride = (case[7], case[8])
    dx = O.conv_dgrad(dy, w, x.shape[1:3], stride, case[9], dtype=np.float64)
    dxb = O.conv_dgrad_bruteforce(dy, w, x.shape[1:3], stride, case[9])
    np.testing.assert_allclose(dx, dxb, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("case", CASES)
def test_adjoint_identities(case):
    x, w, b, dy, P = _rand_case(case, seed=3)
    stride = (case[7], case[8])
    y0 = O.conv_fprop(x, w, None, stride, case[9], dtype=np.float64)
    dx = O.conv_dgrad(dy, w, x.shape[1:3], stride, case[9], dtype=np.float64)
    dw = O.conv_wgrad(x, dy, w.shape[:2], stride, case[9], dtype=np.float64)
    lhs = np.sum(y0 * dy)
    assert abs(lhs - np.sum(x * dx)) < 1e-9 * max(1, abs(lhs))
    assert abs(lhs - np.sum(w * dw)) < 1e-9 * max(1, abs(lhs))


def test_wgrad_finite_differences():
    case = CASES[3]
    x, w, b, dy, P = _rand_case(case, seed=4)
    stride = (case[7], case[8])
    dw = O.conv_wgrad(x, dy, w.shape[:2], stride, case[9], dtype=np.float64)
    r = np.random.RandomState(9)
    for _ in range(10):
        idx = tuple(r.randint(0, n) for n in w.shape)
        wp, wm = w.copy(), w.copy()
        wp[idx] += 1e-6
        wm[idx] -= 1e-6
        lp = np.sum(O.conv_fprop(x, wp, b, stride, case[9], dtype=np.float64) * dy)
        lm = np.sum(O.conv_fprop(x, wm, b, stride, case[9], dtype=np.float64) * dy)
        assert abs((lp - lm) / 2e-6 - dw[idx]) < 1e-6 * max(1.0, abs(dw[idx]))


def test_one_by_one_is_matmul_and_bias_is_zero_input_output():
    r = np.random.RandomState(5)
    x = r.randn(2, 4, 5, 6)
    w = r.randn(1, 1, 6, 7)
    b = r.randn(7)
    y = O.conv_fprop(x, w, b, (1, 1), "valid", dtype=np.float64)
    np.testing.assert_allclose(y.reshape(-1, 7), x.reshape(-1, 6) @ w.reshape(6, 7) + b, rtol=1e-12)
    y0 = O.conv_fprop(np.zeros_like(x), w, b, (1, 1), "valid", dtype=np.float64)
    assert np.all(y0 == b)
    dy = r.randn(2, 4, 5, 7)
    dw = O.conv_wgrad(x, dy, (1, 1), (1, 1), "valid", dtype=np.float64)
    np.testing.assert_allclose(dw.reshape(6, 7), x.reshape(-1, 6).T @ dy.reshape(-1, 7), rtol=1e-12)


def test_dgrad_p0_same_returns_full_tensor():
    # reference returns an empty (S,0,0,C) slice here (classes:119-121); the
    # restatement returns the full gradient.
    r = np.random.RandomState(6)
    dy = r.randn(2, 4, 4, 3)
    w = r.randn(1, 1, 5, 3)
    dx = O.conv_dgrad(dy, w, (4, 4), (1, 1), "same", dtype=np.float64)
    assert dx.shape == (2, 4, 4, 5)
    np.testing.assert_allclose(dx.reshape(-1, 5), dy.reshape(-1, 3) @ w.reshape(5, 3).T, rtol=1e-12)


def test_numpy_reference_quirk_is_not_the_gradient():
    case = CASES[1]
    x, w, b, dy, P = _rand_case(case, seed=7)
    good = O.conv_dgrad(dy, w, x.shape[1:3], (1, 1), "same", dtype=np.float64)
    quirk = O.conv_dgrad(dy, w, x.shape[1:3], (1, 1), "same", dtype=np.float64, numpy_reference_quirk=True)
    assert quirk.shape == good.shape
    assert np.max(np.abs(quirk - good)) > 0.5
    # the quirk is what an overlapping in-place add produces
    from numpy.lib.stride_tricks import as_strided
    S, Ho, Wo, D = dy.shape
    fH, fW, C, _ = w.shape
    pad = np.zeros((S, x.shape[1] + 2, x.shape[2] + 2, C))
    st = pad.strides
    view = as_strided(pad, shape=(S, Ho, Wo, fH, fW, C), strides=(st[0], st[1], st[2], st[1], st[2], st[3]))
    view += np.einsum("shwd,xycd->shwxyc", dy, w)
    np.testing.assert_array_equal(pad[:, 1:-1, 1:-1, :], quirk)


def test_stride2_valid_untouched_border_is_zero():
    # 28x28 input, 3x3 stride 2 valid: row/col 27 never read -> zero gradient
    r = np.random.RandomState(8)
    dy = r.randn(1, 13, 13, 2)
    w = r.randn(3, 3, 3, 2)
    dx = O.conv_dgrad(dy, w, (28, 28), (2, 2), "valid", dtype=np.float64)
    assert dx.shape == (1, 28, 28, 3)
    assert np.all(dx[:, 27] == 0) and np.all(dx[:, :, 27] == 0)


# ---- dense --------------------------------------------------------------------
def test_dense_vs_torch_and_regularisers():
    r = np.random.RandomState(10)
    x = r.randn(7, 5)
    w = r.randn(5, 4)
    w[0, 0] = 0.0
    b = r.randn(1, 4)
    dy = r.randn(7, 4)
    y = O.dense_forward(x, w, b, dtype=np.float64)
    np.testing.assert_allclose(y, F.linear(torch.from_numpy(x), torch.from_numpy(w.T.copy()),
                                           torch.from_numpy(b[0])).numpy(), rtol=1e-12)
    dw, db, dx = O.dense_backward(x, w, b, dy, wl1=0.1, wl2=0.2, bl1=0.3, bl2=0.4, dtype=np.float64)
    sign_w = np.where(w < 0, -1.0, 1.0)   # sign(0) = +1
    sign_b = np.where(b < 0, -1.0, 1.0)
    np.testing.assert_allclose(dw, x.T @ dy + 0.1 * sign_w + 0.4 * w, rtol=1e-12)
    np.testing.assert_allclose(db, dy.sum(0, keepdims=True) + 0.3 * sign_b + 0.8 * b, rtol=1e-12)
    np.testing.assert_allclose(dx, dy @ w.T, rtol=1e-12)
    assert dw[0, 0] == (x.T @ dy)[0, 0] + 0.1


# ---- bf16 helper ---------------------------------------------------------------
def test_bf16_rounding_matches_torch():
    r = np.random.RandomState(11)
    a = (r.randn(10000) * 10.0 ** r.randint(-10, 10, 10000)).astype(np.float32)
    a[:4] = [0.0, -0.0, np.inf, -np.inf]
    want = torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()
    got = O.round_to_bf16(a)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(O.bf16_bits(a), (want.view(np.uint32) >> 16).astype(np.uint16))
