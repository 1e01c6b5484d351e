"""The Adam checks of the step tests (tests/step_checks.py) must refuse wrong updates.  A float32 evaluation of
the update as the GPU kernel makes it passes; no update, a sign flip, a doubled learning rate, a missing bias
correction and a wrong step number are all refused.  Runs on the CPU with NumPy arrays in place of device tensors."""
import numpy as np
import pytest

from tests import step_checks as SC

LR, EPS = 1e-3, 1e-7


class _Layer:
    pass


class _Model:
    pass


def _f32_adam(theta, g, m, v, lr, t, sign=-1.0, correct=True):
    """The kernel's arithmetic: float32 throughout, corrections rounded from float64."""
    f = np.float32
    b1, b2 = f(0.9), f(0.999)
    m = b1 * m + (f(1) - b1) * g
    v = b2 * v + (f(1) - b2) * (g * g)
    c1 = f(1.0 - float(b1) ** (t + 1)) if correct else f(1)
    c2 = f(1.0 - float(b2) ** (t + 1)) if correct else f(1)
    theta = theta + f(sign) * f(lr) * (m / c1) / (np.sqrt(v / c2) + f(EPS))
    return theta.astype(f), m.astype(f), v.astype(f)


def _make(rng, steps_before=0):
    model = _Model()
    model.trainable_layers = []
    for shape, gscale in (((3, 3, 8, 16), 1e-2), ((64, 10), 1.0), ((32,), 1e-9)):
        l = _Layer()
        l.weights = rng.standard_normal(shape).astype(np.float32)
        l.biases = rng.standard_normal(shape[-1:]).astype(np.float32)
        for name, ref in (("weight", l.weights), ("bias", l.biases)):
            setattr(l, name + "_momentums", np.zeros_like(ref))
            setattr(l, name + "_cache", np.zeros_like(ref))
        l.gscale = gscale
        model.trainable_layers.append(l)
    for t in range(steps_before):
        _step(model, rng, t)
    return model


def _step(model, rng, t, lr=LR, step_t=None, **kw):
    for l in model.trainable_layers:
        l.dweights = (rng.standard_normal(l.weights.shape) * l.gscale).astype(np.float32)
        l.dbiases = (rng.standard_normal(l.biases.shape) * l.gscale).astype(np.float32)
        tt = t if step_t is None else step_t
        l.weights, l.weight_momentums, l.weight_cache = _f32_adam(l.weights, l.dweights, l.weight_momentums,
                                                                  l.weight_cache, lr, tt, **kw)
        l.biases, l.bias_momentums, l.bias_cache = _f32_adam(l.biases, l.dbiases, l.bias_momentums, l.bias_cache,
                                                             lr, tt, **kw)


@pytest.mark.parametrize("t", [0, 1, 7])
def test_float32_update_passes_the_own_state_check(t):
    rng = np.random.default_rng(1)
    model = _make(rng, steps_before=t)
    before = SC.snapshot(model)
    _step(model, rng, t)
    SC.check_update_from_own_state(model, before, LR, t, EPS)


@pytest.mark.parametrize("wrong", [dict(sign=1.0), dict(lr=2 * LR), dict(correct=False), dict(step_t=3), "skip",
                                   dict(lr=1.001 * LR)])
def test_wrong_updates_fail_the_own_state_check(wrong):
    rng = np.random.default_rng(2)
    model = _make(rng, steps_before=1)
    before = SC.snapshot(model)
    if wrong == "skip":
        for l in model.trainable_layers:                    # gradients arrive, nothing is updated
            l.dweights = (rng.standard_normal(l.weights.shape) * l.gscale).astype(np.float32)
            l.dbiases = (rng.standard_normal(l.biases.shape) * l.gscale).astype(np.float32)
    else:
        _step(model, rng, 1, **wrong)
    with pytest.raises(AssertionError, match="Adam update off the formula"):
        SC.check_update_from_own_state(model, before, LR, 1, EPS)


def _oracle_side(model, before, rng, rel_noise):
    """What a float64 oracle network would report for the same step: gradients that differ from the GPU's by
    `rel_noise`, and the parameters after its own update."""
    from oracle import oracle as O
    params, grads = [], []
    for l, (sw, sb) in zip(model.trainable_layers, before):
        gw = np.asarray(l.dweights, np.float64) * (1 + rel_noise * rng.standard_normal(l.dweights.shape))
        gb = np.asarray(l.dbiases, np.float64) * (1 + rel_noise * rng.standard_normal(l.dbiases.shape))
        pw = O.adam_update(sw[0], gw, sw[1], sw[2], LR, 0)[0]
        pb = O.adam_update(sb[0], gb, sb[1], sb[2], LR, 0)[0]
        params.append((pw, pb))
        grads.append((gw, gb))
    return params, grads


def test_first_step_passes_against_an_oracle_with_slightly_different_gradients():
    rng = np.random.default_rng(3)
    model = _make(rng)
    before = SC.snapshot(model)
    _step(model, rng, 0)
    params, grads = _oracle_side(model, before, rng, 5e-5)
    seen = SC.check_update_against_oracle(model, before, params, grads, LR, EPS)
    assert len(seen) == 6
    tol = {what: median for what, _, median in seen}
    assert tol["layer 1 weights"] < 2e-4                    # gradients of order 1 >> eps: 1e-5*lr + a rounding of theta
    assert tol["layer 2 weights"] < 2e-4                    # gradients of order 1e-9 << eps: lr*dg/eps is 2e-6*lr


@pytest.mark.parametrize("wrong", [dict(sign=1.0), dict(lr=2 * LR), dict(correct=False), "skip", dict(lr=1.01 * LR)])
def test_wrong_first_steps_fail_against_the_oracle(wrong):
    rng = np.random.default_rng(4)
    model = _make(rng)
    before = SC.snapshot(model)
    if wrong == "skip":
        for l in model.trainable_layers:
            l.dweights = (rng.standard_normal(l.weights.shape) * l.gscale).astype(np.float32)
            l.dbiases = (rng.standard_normal(l.biases.shape) * l.gscale).astype(np.float32)
    else:
        _step(model, rng, 0, **wrong)
    params, grads = _oracle_side(model, before, rng, 5e-5)
    with pytest.raises(AssertionError, match="differ from the oracle"):
        SC.check_update_against_oracle(model, before, params, grads, LR, EPS)


def test_tensors_without_a_gradient_are_left_out_and_an_empty_comparison_is_refused():
    rng = np.random.default_rng(5)
    model = _make(rng)
    before = SC.snapshot(model)
    _step(model, rng, 0)
    params, grads = _oracle_side(model, before, rng, 5e-5)
    grads = [(np.zeros_like(gw), np.zeros_like(gb)) for gw, gb in grads]
    with pytest.raises(AssertionError, match="nothing was compared"):
        SC.check_update_against_oracle(model, before, params, grads, LR, EPS)
