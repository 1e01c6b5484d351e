"""Checks of the Adam update of a training step that a wrong update cannot pass.

Two independent comparisons, both made after every step of the step tests:

``check_update_from_own_state``: the parameters, first and second moments the GPU holds
after the step against the reference's update formula (CNN_classes_cupy.py:702-734,
restated in oracle.adam_update) evaluated in float64 on what the GPU held BEFORE the step
and the gradient the GPU computed.  Every element, tolerance 1e-4*lr on the parameter
change (float32 evaluation of m/(sqrt(v)+eps) and of 1-beta_2) plus one float32 rounding
of the parameter itself.  This pins the update rule at every step, whatever the gradients.

``check_update_against_oracle``: the parameter CHANGE of the first step against the
change the float64 oracle network makes from the same start.  After one step
delta = -lr * f(g), f(g) = g / (|g| + eps), and f is monotone: a gradient within
dg = 1e-4*|g| + 1e-4*rms(g) of the oracle's (the float32 bar of the gradient comparisons)
can move the change by at most lr * max|f(g +- dg) - f(g)|.  That bound, plus 1e-5*lr and
one float32 rounding of the parameter, is the per-element tolerance; where |g| >> eps it
is about 1e-4*lr*eps/|g|, where |g| << eps about lr*dg/eps.  A share of 1e-3 of the
elements may exceed it (gradients that went through a max-pool or ReLU selection that
float32 and float64 decide differently), none may move by more than lr.  The median
tolerance must stay below lr/20, so that the comparison cannot become one that a wrong
update passes.  Tensors whose oracle gradient vanishes identically (a bias in front of a
batch norm) are left to the first check.

A step that did not update, updated with the wrong sign, a wrong learning rate or a wrong
bias correction is off by about lr on most elements (tests/test_step_checks_cpu.py applies
such updates and expects the refusal)."""
import numpy as np

from oracle import oracle as O

_ULP = 2.0 ** -23


def snapshot(model):
    """Host copies of (weights, biases, their Adam moments) of every trainable layer; moments
    that do not exist yet (no step taken) count as zeros, as the reference creates them."""
    snap = []
    for layer in model.trainable_layers:
        if layer.weights is None:
            # a batch norm before its first forward pass: it will create gamma = 1, beta = 0 over the channels
            # it then sees (CNN_classes_cupy.py:453-460); the checks fill the shapes in from the gradients
            snap.append(None)
            continue
        w, b = np.asarray(layer.weights, dtype=np.float64), np.asarray(layer.biases, dtype=np.float64)
        if hasattr(layer, "weight_cache"):
            mw, vw = np.asarray(layer.weight_momentums, np.float64), np.asarray(layer.weight_cache, np.float64)
            mb, vb = np.asarray(layer.bias_momentums, np.float64), np.asarray(layer.bias_cache, np.float64)
        else:
            mw, vw, mb, vb = np.zeros_like(w), np.zeros_like(w), np.zeros_like(b), np.zeros_like(b)
        snap.append(((w, mw, vw), (b, mb, vb)))
    return snap


def _lazy(entry, layer):
    """A snapshot entry; for a layer that had no parameters yet, the values its first forward pass gives them."""
    if entry is not None:
        return entry
    w, b = np.ones(np.asarray(layer.weights).shape), np.zeros(np.asarray(layer.biases).shape)
    return ((w, np.zeros_like(w), np.zeros_like(w)), (b, np.zeros_like(b), np.zeros_like(b)))


def update_errors(theta0, g, m0, v0, theta1, m1, v1, lr, iterations, eps=1e-7, beta1=0.9, beta2=0.999):
    """Worst err/tol of (theta1, m1, v1) against the formula applied in float64 to (theta0, g, m0, v0)."""
    theta0, g, m0, v0 = (np.asarray(a, np.float64) for a in (theta0, g, m0, v0))
    g = g.reshape(theta0.shape)
    want_t, want_m, want_v = O.adam_update(theta0, g, m0, v0, lr, iterations, beta1, beta2, eps)
    got_t, got_m, got_v = (np.asarray(a, np.float64).reshape(theta0.shape) for a in (theta1, m1, v1))
    e_t = np.abs((got_t - theta0) - (want_t - theta0)) / (1e-4 * lr + _ULP * np.abs(want_t))
    # (the absolute floor covers float32 underflow of the moments of vanishing gradients; the first moment's
    # two terms may cancel, so its tolerance follows the terms, not the sum)
    e_m = np.abs(got_m - want_m) / (1e-36 + 1e-5 * (beta1 * np.abs(m0) + (1 - beta1) * np.abs(g)))
    e_v = np.abs(got_v - want_v) / (1e-36 + 1e-4 * np.abs(want_v))
    return float(e_t.max()), float(e_m.max()), float(e_v.max())


def check_update_from_own_state(model, before, lr, iterations, eps=1e-7):
    """`before` = snapshot(model) taken before the step; the layers now hold the step's gradients and results."""
    for i, (layer, entry) in enumerate(zip(model.trainable_layers, before)):
        sw, sb = _lazy(entry, layer)
        for name, (t0, m0, v0), g, t1, m1, v1 in (
                ("weights", sw, layer.dweights, layer.weights, layer.weight_momentums, layer.weight_cache),
                ("biases", sb, layer.dbiases, layer.biases, layer.bias_momentums, layer.bias_cache)):
            e = update_errors(t0, np.asarray(g), m0, v0, np.asarray(t1), np.asarray(m1), np.asarray(v1),
                              lr, iterations, eps)
            assert max(e) <= 1.0, "layer %d %s: Adam update off the formula, err/tol (theta, m, v) = %r" % (i, name, e)


def delta_errors(theta0, theta_gpu, theta_oracle, g_oracle, lr, eps=1e-7):
    """(share of elements outside the tolerance, median tolerance / lr, largest |change| / lr)."""
    theta0 = np.asarray(theta0, np.float64)
    d_gpu = np.asarray(theta_gpu, np.float64).reshape(theta0.shape) - theta0
    d_ref = np.asarray(theta_oracle, np.float64).reshape(theta0.shape) - theta0
    g = np.asarray(g_oracle, np.float64).reshape(theta0.shape)
    dg = 1e-4 * np.abs(g) + 1e-4 * float(np.sqrt(np.mean(g * g)))
    f = lambda a: a / (np.abs(a) + eps)
    reach = np.maximum(np.abs(f(g + dg) - f(g)), np.abs(f(g - dg) - f(g)))
    tol = lr * (reach + 1e-5) + _ULP * np.abs(theta0)
    outside = float(np.mean(np.abs(d_gpu - d_ref) > tol))
    return outside, float(np.median(tol) / lr), float(np.max(np.abs(d_gpu)) / lr)


def check_update_against_oracle(model, before, oracle_params, oracle_grads, lr, eps=1e-7):
    """First step only: `before` = snapshot(model) before it, `oracle_params` / `oracle_grads` the oracle
    network's parameters after and gradients of the same step.  Returns what was measured per tensor."""
    seen = []
    for i, (layer, entry) in enumerate(zip(model.trainable_layers, before)):
        sw, sb = _lazy(entry, layer)
        for j, (name, (t0, _, _), t1) in enumerate((("weights", sw, layer.weights), ("biases", sb, layer.biases))):
            g = np.asarray(oracle_grads[i][j], np.float64)
            if np.linalg.norm(g) <= 1e-12:
                continue
            outside, median_tol, largest = delta_errors(t0, np.asarray(t1), oracle_params[i][j], g, lr, eps)
            what = "layer %d %s" % (i, name)
            assert median_tol <= 0.05, "%s: median tolerance %.3g * lr is no check" % (what, median_tol)
            assert outside <= 1e-3, "%s: %.4f of the parameter changes differ from the oracle's" % (what, outside)
            assert largest <= 1.0 + 1e-4, "%s: a first Adam step moved an element by %.6g * lr" % (what, largest)
            seen.append((what, outside, median_tol))
    assert seen, "nothing was compared"
    return seen
