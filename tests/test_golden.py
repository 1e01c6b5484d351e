"""The known answers the reference's notebooks hold for this path, kept as data in
tests/golden/notebook_known_answers.json: the CPU oracle must reproduce them (no GPU),
and so must the library through its C ABI (GPU)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "notebook_known_answers.json")) as f:
    GOLDEN = json.load(f)["cases"]


def _oracle_backend():
    return {
        "fprop": lambda x, w, b, s, p: O.conv_fprop(x, w, b, s, p, dtype=np.float64),
        "dgrad": lambda dy, w, hw, s, p: O.conv_dgrad(dy, w, hw, s, p, dtype=np.float64),
        "maxpool": lambda x: (lambda y, i: (y, O.maxpool_backward(y, i, x.shape)))(*O.maxpool_forward(x)),
        "avgpool": lambda x: (lambda y: (y, O.avgpool_backward(y, x.shape)))(O.avgpool_forward(x)),
    }


def _gpu_backend():
    import aether
    from tests import abi

    def pool(kind):
        def run(x):
            layer = aether.Pooling(pooling_type=kind)
            y = layer.forward(x, True)
            layer.backward(y)
            return y.get(), layer.dinputs.get()
        return run

    return {
        "fprop": lambda x, w, b, s, p: abi.fprop(x.astype(np.float32), w.astype(np.float32),
                                                None if b is None else b.astype(np.float32), s, p),
        "dgrad": lambda dy, w, hw, s, p: abi.dgrad(dy.astype(np.float32), w.astype(np.float32),
                                                   (dy.shape[0], hw[0], hw[1], w.shape[2]), s, p),
        "maxpool": pool("max"),
        "avgpool": pool("average"),
    }


def _check(case, be):
    op = case["op"]
    strides = tuple(case.get("strides", (1, 1)))
    if op == "conv_fprop":
        x = np.array(case["x_hw"], dtype=np.float64)[None, :, :, None]
        w = np.array(case["w_hw"], dtype=np.float64)[:, :, None, None]
        y = be["fprop"](x, w, None, strides, case["padding"])
        assert np.array_equal(np.asarray(y)[0, :, :, 0], np.array(case["y_hw"], dtype=np.float64))
    elif op == "conv_fprop_const":
        x = np.full(case["x_shape"], case["x_value"], dtype=np.float64)
        w = np.empty(case["w_shape"], dtype=np.float64)
        for d, v in enumerate(case["w_value_per_filter"]):
            w[..., d] = v
        y = np.asarray(be["fprop"](x, w, np.zeros(w.shape[3]), strides, case["padding"]))
        assert list(y.shape) == case["y_shape"]
        for d, v in enumerate(case["y_value_per_filter"]):
            assert np.all(y[..., d] == v)
    elif op == "conv_dgrad_row":
        H, W = case["x_hw_shape"]
        dy = np.zeros((1, H, W, 1))
        dy[0, 0, :, 0] = case["dy_first_row"]
        w = np.full((3, 3, 1, 1), case["w_value"], dtype=np.float64)
        dx = np.asarray(be["dgrad"](dy, w, (H, W), strides, case["padding"]))
        assert np.array_equal(dx[0, 0, :, 0], case["dx_first_row"])
    elif op in ("maxpool", "avgpool"):
        x = np.array(case["x_hw"], dtype=np.float32)[None, :, :, None]
        y, dx = be[op](x)
        assert np.array_equal(np.asarray(y)[0, :, :, 0], np.array(case["pooled"], dtype=np.float32))
        assert np.array_equal(np.asarray(dx)[0, :, :, 0], np.array(case["dx_of_pooled"], dtype=np.float32))
    else:
        raise AssertionError("unknown golden op %r" % op)


@pytest.mark.parametrize("case", GOLDEN, ids=lambda c: c["name"])
def test_oracle_reproduces_the_reference_known_answers(case):
    _check(case, _oracle_backend())


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLDEN, ids=lambda c: c["name"])
def test_library_reproduces_the_reference_known_answers(case):
    _check(case, _gpu_backend())
