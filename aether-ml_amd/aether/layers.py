"""Layer, loss and optimizer classes with the reference's names, constructor
signatures and attributes (CNN/models/CNN_classes_cupy.py), running on
libaether_hip.so.  ``forward(inputs, training)`` sets ``.output``,
``backward(dvalues)`` sets ``.dinputs`` (+ ``.dweights`` / ``.dbiases``); all of
these are DeviceTensors in MI355X HBM.  Inputs may be NumPy arrays (uploaded) or
DeviceTensors.

Departures from the reference, each deliberate:
  * everything is float32 on the device (the reference's Dense weights are
    float64 by accident of ``cp.random.randn``);
  * ``Conv_Layer.dinputs`` is the full gradient also when the pad is 0 under
    "same" (the reference slices ``[:, 0:-0]`` to an empty array, :149-151);
  * ``Conv_Layer.set_parameters`` refreshes the ``weights`` alias (:159-161 does not);
  * ``Pooling(padding="same")`` raises ValueError (the reference reads ``H_out``
    before assigning it, :226-228).
"""
import os

import numpy as np

from . import _lib
from .tensor import DeviceTensor, as_device

_F32 = np.float32


def _L():
    return _lib.lib()


def _ck(rc):
    _lib.check(rc)


_recording = [False]        # a training step is being recorded (Model sets it around the capture)
_recorded_masks = []        # while recording: (dropout layer, the device buffer its recorded kernels read the mask from)


def _wants_bf16(layer):
    """True for a convolution that runs on bf16 inputs: the kernel that produces its input
    (or its upstream gradient) then leaves a bfloat16 copy beside the float32 tensor."""
    return isinstance(layer, Conv_Layer) and layer.precision == "bf16"


def _twin(t):
    """Attach an empty bfloat16 copy to a float32 tensor and return it."""
    t._bf16 = DeviceTensor(t.shape, np.uint16)
    return t._bf16


# ----------------------------------------------------------------------------------
# Conv_Layer  (CNN_classes_cupy.py:37-161)
# ----------------------------------------------------------------------------------
class Conv_Layer:
    def __init__(self, input_shape, num_filters=1, filter_size=(3, 3), strides=(1, 1), padding="same"):
        self.input_shape = input_shape
        self.num_filters = num_filters
        self.filter_size = filter_size
        self.strides = strides
        self.padding = padding
        self.biases = DeviceTensor.zeros(self.num_filters)
        self.weight_regularizer_l1 = 0
        self.weight_regularizer_l2 = 0
        self.bias_regularizer_l1 = 0
        self.bias_regularizer_l2 = 0
        input_depth = input_shape[-1]
        n = self.filter_size[0] * self.filter_size[1] * input_depth
        std = np.sqrt(_F32(2.0 / n))
        # He initialisation from the legacy global RNG, as the reference (:61-66)
        w = np.random.randn(filter_size[0], filter_size[1], input_depth, num_filters).astype(_F32) * std
        self.filter_weights = DeviceTensor.from_numpy(w, _F32)
        self.weights = self.filter_weights
        # "fp32" (reference arithmetic) or "bf16" (bf16 inputs, fp32 accumulate)
        self.precision = os.environ.get("AETHER_PRECISION", "fp32")

    def _geometry(self, H_in, W_in):
        fH, fW = self.filter_size
        sH, sW = self.strides
        P = (fH - 1) // 2 if self.padding == "same" else 0
        H_out = int((H_in + 2 * P - fH) / sH + 1)
        W_out = int((W_in + 2 * P - fW) / sW + 1)
        return P, H_out, W_out

    def _dims(self, S, H, W, C):
        fH, fW = self.filter_size
        sH, sW = self.strides
        P = (fH - 1) // 2 if self.padding == "same" else 0
        return (S, H, W, C, self.num_filters, fH, fW, sH, sW, P, P)

    @staticmethod
    def _bf16(t):
        """The tensor's bfloat16 copy: the one its producing kernel left beside it, else a cast."""
        if t._bf16 is not None:
            return t._bf16
        out = DeviceTensor(t.shape, np.uint16)
        _ck(_L().aeth_cast_f32_to_bf16(t.ptr, out.ptr, t.size))
        return out

    def _filter_bf16(self):
        """bfloat16 filter, cast once per version of the weights (the optimizer and
        set_parameters change the version).  While a step is being recorded the cast always
        runs, so that it is part of the recording."""
        w = self.filter_weights
        # keyed on the tensor object, not its address: the allocator hands a freed block's address out again
        fresh = getattr(self, "_w16_src", None) is w and getattr(self, "_w16_version", None) == w._version
        if _recording[0] or not fresh:
            out = DeviceTensor(w.shape, np.uint16)
            _ck(_L().aeth_cast_f32_to_bf16(w.ptr, out.ptr, w.size))
            self._w16, self._w16_src, self._w16_version = out, w, w._version
        return self._w16

    def forward(self, inputs, training):
        inputs = as_device(inputs, _F32)
        if inputs.ndim != 4:
            raise ValueError(f"Expected a 4D tensor, got {inputs.ndim} instead.")
        S, H_in, W_in, D_in = inputs.shape
        if D_in != self.filter_weights.shape[2]:
            raise ValueError(f"Expected {self.filter_weights.shape[2]} input channels, got {D_in}.")
        P, H_out, W_out = self._geometry(H_in, W_in)
        self.output = DeviceTensor((S, H_out, W_out, self.num_filters), _F32)
        dims = self._dims(S, H_in, W_in, D_in)
        if self.precision == "bf16":
            self._x_bf16 = self._bf16(inputs)
            w16 = self._filter_bf16()
            _ck(_L().aeth_conv_fprop_bf16(self._x_bf16.ptr, w16.ptr, self.biases.ptr, self.output.ptr, *dims))
        else:
            _ck(_L().aeth_conv_fprop_f32(inputs.ptr, self.filter_weights.ptr, self.biases.ptr,
                                         self.output.ptr, *dims))
        self.inputs = inputs
        return self.output

    def backward(self, dvalues):
        dvalues = as_device(dvalues, _F32)
        S, H_in, W_in, C_in = self.inputs.shape
        dims = self._dims(S, H_in, W_in, C_in)
        self.dbiases = DeviceTensor(self.biases.shape, _F32)
        self.dweights = DeviceTensor(self.filter_weights.shape, _F32)
        self.dinputs = DeviceTensor(self.inputs.shape, _F32)
        if self.precision == "bf16":
            dy16 = self._bf16(dvalues)
            w16 = self._filter_bf16()
            _ck(_L().aeth_conv_wgrad_bf16(self._x_bf16.ptr, dy16.ptr, self.dweights.ptr, self.dbiases.ptr, *dims))
            _ck(_L().aeth_conv_dgrad_bf16(dy16.ptr, w16.ptr, self.dinputs.ptr, *dims))
        else:
            # filter / bias gradient and input gradient in one call (one launch for both where neither fills the GPU)
            _ck(_L().aeth_conv_bwd_f32(self.inputs.ptr, dvalues.ptr, self.filter_weights.ptr, self.dweights.ptr,
                                       self.dbiases.ptr, self.dinputs.ptr, *dims))
        return self.dinputs

    def get_parameters(self):
        return self.filter_weights, self.biases

    def set_parameters(self, weights, biases):
        self.filter_weights = as_device(weights, _F32)
        self.biases = as_device(biases, _F32).reshape(-1)
        self.weights = self.filter_weights


# ----------------------------------------------------------------------------------
# Pooling  (CNN_classes_cupy.py:204-312)
# ----------------------------------------------------------------------------------
class Pooling:
    def __init__(self, filter_size=(2, 2), strides=(2, 2), padding="valid", pooling_type="max"):
        self.filter_size = filter_size
        self.strides = strides
        self.padding = padding
        self.pooling_type = pooling_type

    def forward(self, inputs, training):
        if _take_prefilled(self, inputs):       # a Batch_Norm two layers up has done this pass
            return self.output
        self._fused_relu = self._fused_bn = None
        inputs = as_device(inputs, _F32)
        if inputs.ndim != 4:
            raise ValueError(f"Expected a 4D tensor, got {inputs.ndim} instead.")
        S, H_in, W_in, C = inputs.shape
        fH, fW = self.filter_size
        sH, sW = self.strides
        if self.padding == "valid":
            H_out = int(np.floor((H_in - fH) / sH + 1))
            W_out = int(np.floor((W_in - fW) / sW + 1))
        elif self.padding == "same":
            raise ValueError("Pooling with padding == same is not supported")
        else:
            raise ValueError(f"Expected padding == valid or same, recieved {self.padding} instead")
        self.inputs = inputs
        self.output = DeviceTensor((S, H_out, W_out, C), _F32)
        if self.pooling_type == "max":
            self.max_indicies = DeviceTensor((S, H_out, W_out, C), np.uint8)
            _ck(_L().aeth_maxpool_fwd_f32(inputs.ptr, self.output.ptr, self.max_indicies.ptr,
                                          S, H_in, W_in, C, fH, fW, sH, sW))
        elif self.pooling_type == "average":
            _ck(_L().aeth_avgpool_fwd_f32(inputs.ptr, self.output.ptr, S, H_in, W_in, C, fH, fW, sH, sW))
        else:
            raise ValueError(f"Expected pooling_type == max or average, recieved {self.pooling_type} instead")
        return self.output

    def backward(self, dvalues):
        dvalues = as_device(dvalues, _F32)
        S, H_in, W_in, C = self.inputs.shape
        fH, fW = self.filter_size
        sH, sW = self.strides
        self.dinputs = DeviceTensor(self.inputs.shape, _F32)
        relu = getattr(self, "_fused_relu", None)
        if relu is not None:
            # the forward pass of this block was fused: one kernel for this layer's and the
            # activation's backward pass (the activation then finds its dinputs in place),
            # which also takes the batch norm's column sums when the channel count allows it
            relu.dinputs = DeviceTensor(self.inputs.shape, _F32)
            bn = getattr(self, "_fused_bn", None)
            c4 = C // 4
            if bn is not None and 256 % c4 == 0:
                bn.dinputs = DeviceTensor(self.inputs.shape, _F32)
                bn.dweights = DeviceTensor(C, _F32)
                bn.dbiases = DeviceTensor(C, _F32)
                head = (dvalues.ptr, self.max_indicies.ptr, relu.inputs.ptr, bn.inputs.ptr, bn.gamma.ptr,
                        bn.batch_mean.ptr, bn.batch_invstd.ptr, self.dinputs.ptr, relu.dinputs.ptr, bn.dinputs.ptr)
                tail = (bn.dweights.ptr, bn.dbiases.ptr, S, H_in, W_in, C, _relu_alpha(relu))
                if _wants_bf16(getattr(bn, "prev", None)):
                    _ck(_L().aeth_maxpool2_relu_bn_bwd_twin_f32(*head, _twin(bn.dinputs).ptr, *tail))
                else:
                    _ck(_L().aeth_maxpool2_relu_bn_bwd_f32(*head, *tail))
                bn._bwd_prefilled_for = relu.dinputs
            else:
                _ck(_L().aeth_maxpool2_relu_bwd_f32(dvalues.ptr, self.max_indicies.ptr, relu.inputs.ptr,
                                                    self.dinputs.ptr, relu.dinputs.ptr, S, H_in, W_in, C,
                                                    _relu_alpha(relu)))
            relu._bwd_prefilled_for = self.dinputs
            return self.dinputs
        if self.pooling_type == "max":
            _ck(_L().aeth_maxpool_bwd_f32(dvalues.ptr, self.max_indicies.ptr, self.dinputs.ptr,
                                          S, H_in, W_in, C, fH, fW, sH, sW))
        elif self.pooling_type == "average":
            _ck(_L().aeth_avgpool_bwd_f32(dvalues.ptr, self.dinputs.ptr, S, H_in, W_in, C, fH, fW, sH, sW))
        return self.dinputs


# ----------------------------------------------------------------------------------
# Layer_Dense  (CNN_classes_cupy.py:315-362)
# ----------------------------------------------------------------------------------
class Layer_Dense:
    def __init__(self, n_inputs, n_neurons, weight_regularizer_l1=0, bias_regularizer_l1=0,
                 weight_regularizer_l2=0, bias_regularizer_l2=0):
        w = .01 * np.random.randn(n_inputs, n_neurons) * np.sqrt(2.0 / n_inputs)
        self.weights = DeviceTensor.from_numpy(w, _F32)
        self.biases = DeviceTensor.zeros((1, n_neurons))
        self.weight_regularizer_l1 = weight_regularizer_l1
        self.weight_regularizer_l2 = weight_regularizer_l2
        self.bias_regularizer_l1 = bias_regularizer_l1
        self.bias_regularizer_l2 = bias_regularizer_l2

    def forward(self, inputs, training):
        inputs = as_device(inputs, _F32)
        if inputs.ndim != 2 or inputs.shape[1] != self.weights.shape[0]:
            raise ValueError(f"shapes {inputs.shape} and {self.weights.shape} not aligned")
        self.inputs = inputs
        M = inputs.shape[0]
        n_in, n_out = self.weights.shape
        self.output = DeviceTensor((M, n_out), _F32)
        act = self._neighbour("next")
        if act is not None and not _wants_bf16(getattr(act, "next", None)):
            # the ReLU / Leaky_ReLU behind this layer in the same call (it then finds its output in place): where K is
            # split over workgroups, the reduction of the split writes both tensors
            act.inputs = self.output
            act.output = DeviceTensor((M, n_out), _F32)
            _ck(_L().aeth_dense_fprop_act_f32(inputs.ptr, self.weights.ptr, self.biases.ptr, self.output.ptr,
                                              act.output.ptr, _relu_alpha(act), M, n_in, n_out))
            act._prefilled_for = self.output
            return self.output
        _ck(_L().aeth_dense_fprop_f32(inputs.ptr, self.weights.ptr, self.biases.ptr, self.output.ptr,
                                      M, n_in, n_out))
        return self.output

    def _neighbour(self, side):
        """The ReLU / Leaky_ReLU directly behind ("next") or in front of ("prev") this layer, if the model has linked
        one there and AETHER_FUSE_DENSE is not 0."""
        layer = getattr(self, side, None)
        if isinstance(layer, (ReLU, Leaky_ReLU)) and os.environ.get("AETHER_FUSE_DENSE", "1") != "0":
            return layer
        return None

    def backward(self, dvalues):
        dvalues = as_device(dvalues, _F32)
        M = self.inputs.shape[0]
        n_in, n_out = self.weights.shape
        self.dweights = DeviceTensor(self.weights.shape, _F32)
        self.dbiases = DeviceTensor((1, n_out), _F32)
        self.dinputs = DeviceTensor(self.inputs.shape, _F32)
        # the three products of the backward pass in one call, with the backward pass of a ReLU / Leaky_ReLU in front of
        # this layer on the way (that layer then finds its dinputs in place)
        act = self._neighbour("prev")
        if act is not None and getattr(act, "output", None) is self.inputs and getattr(act, "inputs", None) is not None \
                and act.inputs.shape == self.inputs.shape:
            act.dinputs = DeviceTensor(self.inputs.shape, _F32)
            act_in, act_dx = act.inputs.ptr, act.dinputs.ptr
        else:
            act, act_in, act_dx = None, None, None
        _ck(_L().aeth_dense_bwd_f32(self.inputs.ptr, dvalues.ptr, self.weights.ptr, self.dweights.ptr, self.dbiases.ptr,
                                    self.dinputs.ptr, act_in, act_dx, _relu_alpha(act) if act is not None else 0.0,
                                    M, n_in, n_out))
        if act is not None:
            act._bwd_prefilled_for = self.dinputs
        if self.weight_regularizer_l1 > 0:
            _ck(_L().aeth_l1_grad_f32(self.weight_regularizer_l1, self.weights.ptr, self.dweights.ptr,
                                      self.weights.size))
        if self.weight_regularizer_l2 > 0:
            _ck(_L().aeth_axpy_f32(2 * self.weight_regularizer_l2, self.weights.ptr, self.dweights.ptr,
                                   self.weights.size))
        if self.bias_regularizer_l1 > 0:
            _ck(_L().aeth_l1_grad_f32(self.bias_regularizer_l1, self.biases.ptr, self.dbiases.ptr,
                                      self.biases.size))
        if self.bias_regularizer_l2 > 0:
            _ck(_L().aeth_axpy_f32(2 * self.bias_regularizer_l2, self.biases.ptr, self.dbiases.ptr,
                                   self.biases.size))

    def get_parameters(self):
        return self.weights, self.biases

    def set_parameters(self, weights, biases):
        self.weights = as_device(weights, _F32)
        b = as_device(biases, _F32)
        self.biases = b.reshape(1, b.size)


# ----------------------------------------------------------------------------------
# Dropout  (CNN_classes_cupy.py:364-404).  Masks are drawn on the host from the
# legacy global RNG, exactly as the reference draws them, and multiplied on the GPU.
# Assigning ``fixed_mask`` (already divided by the keep probability) replaces the draw.
# ----------------------------------------------------------------------------------
class Layer_Dropout:
    def __init__(self, rate):
        self.rate = 1 - rate
        self.fixed_mask = None

    def host_mask(self, shape):
        """This step's mask on the host: Bernoulli(keep) / keep from the legacy global RNG (:375-376), or `fixed_mask`."""
        if self.fixed_mask is not None:
            return np.ascontiguousarray(np.broadcast_to(np.asarray(self.fixed_mask, dtype=_F32), shape))
        return (np.random.binomial(1, self.rate, size=shape) / self.rate).astype(_F32)

    def forward(self, inputs, training):
        inputs = as_device(inputs, _F32)
        self.inputs = inputs
        if not training:
            self.output = inputs.copy()
            return self.output
        if _recording[0]:
            # the recorded kernels read the mask from this buffer; Model fills it before every replay
            self.binary_mask = DeviceTensor(inputs.shape, _F32)
            _recorded_masks.append((self, self.binary_mask))
        else:
            self.binary_mask = DeviceTensor.from_numpy(self.host_mask(inputs.shape), _F32)
        self.output = DeviceTensor(inputs.shape, _F32)
        _ck(_L().aeth_mul_mask_f32(inputs.ptr, self.binary_mask.ptr, self.output.ptr, inputs.size, inputs.size))
        return self.output

    def backward(self, dvalues):
        dvalues = as_device(dvalues, _F32)
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        _ck(_L().aeth_mul_mask_f32(dvalues.ptr, self.binary_mask.ptr, self.dinputs.ptr, dvalues.size, dvalues.size))


class Layer_Dropout_Spatial:
    def __init__(self, rate):
        self.rate = rate
        self.keep_prob = 1 - rate
        self.fixed_mask = None

    def host_mask(self, shape):
        """One draw per channel, shared by the whole batch (:397-398), or `fixed_mask`."""
        if self.fixed_mask is not None:
            return np.asarray(self.fixed_mask, dtype=_F32).reshape(shape)
        return (np.random.binomial(1, self.keep_prob, size=shape) / self.keep_prob).astype(_F32)

    def forward(self, inputs, training):
        inputs = as_device(inputs, _F32)
        self.inputs = inputs
        if not training:
            self.output = inputs.copy()
            return self.output
        C = inputs.shape[-1]
        if _recording[0]:
            self.channel_mask = DeviceTensor((1, 1, 1, C), _F32)    # filled by Model before every replay
            _recorded_masks.append((self, self.channel_mask))
        else:
            self.channel_mask = DeviceTensor.from_numpy(self.host_mask((1, 1, 1, C)), _F32)
        self.output = DeviceTensor(inputs.shape, _F32)
        _ck(_L().aeth_mul_mask_f32(inputs.ptr, self.channel_mask.ptr, self.output.ptr, inputs.size, C))
        return self.output

    def backward(self, dvalues):
        dvalues = as_device(dvalues, _F32)
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        _ck(_L().aeth_mul_mask_f32(dvalues.ptr, self.channel_mask.ptr, self.dinputs.ptr, dvalues.size,
                                   self.channel_mask.size))


# ----------------------------------------------------------------------------------
# ReLU / Leaky_ReLU  (CNN_classes_cupy.py:406-428)
# ----------------------------------------------------------------------------------
def _take_prefilled(layer, inputs):
    """True when a fused kernel further up has already produced this layer's output
    for exactly this input tensor (see Batch_Norm._forward_block)."""
    if getattr(layer, "_prefilled_for", None) is inputs and inputs is not None:
        layer._prefilled_for = None
        return True
    layer._prefilled_for = None
    return False


def _take_bwd_prefilled(layer, dvalues):
    if getattr(layer, "_bwd_prefilled_for", None) is dvalues and dvalues is not None:
        layer._bwd_prefilled_for = None
        return True
    layer._bwd_prefilled_for = None
    return False


def _relu_alpha(layer):
    return float(layer.alpha) if isinstance(layer, Leaky_ReLU) else 0.0


class ReLU:
    def forward(self, inputs, training):
        if _take_prefilled(self, inputs):
            return self.output
        inputs = as_device(inputs, _F32)
        self.inputs = inputs
        self.output = DeviceTensor(inputs.shape, _F32)
        if _wants_bf16(getattr(self, "next", None)):
            _ck(_L().aeth_relu_fwd_twin_f32(inputs.ptr, self.output.ptr, _twin(self.output).ptr, 0.0, inputs.size))
        else:
            _ck(_L().aeth_relu_fwd_f32(inputs.ptr, self.output.ptr, 0.0, inputs.size))
        return self.output

    def backward(self, dvalues):
        if _take_bwd_prefilled(self, dvalues):
            return
        dvalues = as_device(dvalues, _F32)
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        _ck(_L().aeth_relu_bwd_f32(self.inputs.ptr, dvalues.ptr, self.dinputs.ptr, 0.0, dvalues.size))


class Leaky_ReLU:
    def __init__(self, alpha=0.01):
        self.alpha = alpha

    def forward(self, inputs, training):
        if _take_prefilled(self, inputs):
            return self.output
        inputs = as_device(inputs, _F32)
        self.inputs = inputs
        self.output = DeviceTensor(inputs.shape, _F32)
        if _wants_bf16(getattr(self, "next", None)):
            _ck(_L().aeth_relu_fwd_twin_f32(inputs.ptr, self.output.ptr, _twin(self.output).ptr, self.alpha, inputs.size))
        else:
            _ck(_L().aeth_relu_fwd_f32(inputs.ptr, self.output.ptr, self.alpha, inputs.size))
        return self.output

    def backward(self, dvalues):
        if _take_bwd_prefilled(self, dvalues):
            return
        dvalues = as_device(dvalues, _F32)
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        _ck(_L().aeth_relu_bwd_f32(self.inputs.ptr, dvalues.ptr, self.dinputs.ptr, self.alpha, dvalues.size))


# ----------------------------------------------------------------------------------
# Batch_Norm  (CNN_classes_cupy.py:430-526)
# ----------------------------------------------------------------------------------
class Batch_Norm:
    def __init__(self, epsilon=1e-5, momentum=0.9, n_features=None):
        self.epsilon = epsilon
        self.momentum = momentum
        if n_features is not None:
            self.gamma = DeviceTensor.full(n_features, 1.0)
            self.beta = DeviceTensor.zeros(n_features)
        else:
            self.gamma = None
            self.beta = None
        self.weights = self.gamma
        self.biases = self.beta
        self.running_mean = None
        self.running_var = None
        self.weight_regularizer_l1 = 0
        self.weight_regularizer_l2 = 0
        self.bias_regularizer_l1 = 0
        self.bias_regularizer_l2 = 0

    def _lazy_init(self, C):
        if self.gamma is None:
            self.gamma = DeviceTensor.full(C, 1.0)
            self.beta = DeviceTensor.zeros(C)
            self.weights = self.gamma
            self.biases = self.beta
        if self.running_mean is None:
            self.running_mean = DeviceTensor.zeros(C)
            self.running_var = DeviceTensor.full(C, 1.0)

    def forward(self, inputs, training):
        inputs = as_device(inputs, _F32)
        self.inputs = inputs
        C = inputs.shape[-1]
        self._lazy_init(C)
        rows = inputs.size // C
        self.output = DeviceTensor(inputs.shape, _F32)
        if training:
            self.batch_mean = DeviceTensor(C, _F32)
            self.batch_invstd = DeviceTensor(C, _F32)
            block = self._block_tail(inputs)
            if block is not None:
                self._forward_block(inputs, *block)
            else:
                _ck(_L().aeth_bn_fwd_train_f32(inputs.ptr, self.gamma.ptr, self.beta.ptr, self.running_mean.ptr,
                                               self.running_var.ptr, self.batch_mean.ptr, self.batch_invstd.ptr,
                                               self.output.ptr, rows, C, self.epsilon, self.momentum))
            # the reference's running statistics take the keepdims shape after a
            # training step (:475-476); keep that shape for get_parameters()
            keep = (1,) * (inputs.ndim - 1) + (C,)
            if self.running_mean.shape != keep:
                self.running_mean = self.running_mean.reshape(keep)
                self.running_var = self.running_var.reshape(keep)
        else:
            _ck(_L().aeth_bn_fwd_infer_f32(inputs.ptr, self.gamma.ptr, self.beta.ptr, self.running_mean.ptr,
                                           self.running_var.ptr, self.output.ptr, rows, C, self.epsilon))
        return self.output

    # The usual convolution block is Batch_Norm -> ReLU / Leaky_ReLU -> Pooling(max, 2x2, stride 2).
    # In training the three layers run as one pass over the tensor that writes all three
    # outputs; the two layers behind find theirs in place when the model calls them with
    # this layer's output.  AETHER_FUSE_BLOCK=0 keeps the layers apart.
    def _block_tail(self, inputs):
        if os.environ.get("AETHER_FUSE_BLOCK", "1") == "0" or inputs.ndim != 4:
            return None
        act = getattr(self, "next", None)
        pool = getattr(act, "next", None)
        if not isinstance(act, (ReLU, Leaky_ReLU)) or not isinstance(pool, Pooling):
            return None
        if (pool.pooling_type != "max" or pool.padding != "valid" or tuple(pool.filter_size) != (2, 2)
                or tuple(pool.strides) != (2, 2)):
            return None
        S, H, W, C = inputs.shape
        if H % 2 or W % 2 or C % 4:
            return None
        return act, pool

    def _forward_block(self, inputs, act, pool):
        S, H, W, C = inputs.shape
        act.inputs = self.output
        act.output = DeviceTensor(inputs.shape, _F32)
        pool.inputs = act.output
        pool.output = DeviceTensor((S, H // 2, W // 2, C), _F32)
        pool.max_indicies = DeviceTensor((S, H // 2, W // 2, C), np.uint8)
        head = (inputs.ptr, self.gamma.ptr, self.beta.ptr, self.running_mean.ptr, self.running_var.ptr,
                self.batch_mean.ptr, self.batch_invstd.ptr, self.output.ptr, act.output.ptr, pool.output.ptr)
        tail = (pool.max_indicies.ptr, S, H, W, C, self.epsilon, self.momentum, _relu_alpha(act))
        if _wants_bf16(getattr(pool, "next", None)):
            _ck(_L().aeth_bn_relu_maxpool2_fwd_twin_f32(*head, _twin(pool.output).ptr, *tail))
        else:
            _ck(_L().aeth_bn_relu_maxpool2_fwd_f32(*head, *tail))
        act._prefilled_for = self.output
        pool._prefilled_for = act.output
        pool._fused_relu = act
        pool._fused_bn = self

    def backward(self, dvalues):
        if _take_bwd_prefilled(self, dvalues):
            return self.dinputs
        dvalues = as_device(dvalues, _F32)
        C = self.inputs.shape[-1]
        rows = self.inputs.size // C
        self.dinputs = DeviceTensor(self.inputs.shape, _F32)
        self.dweights = DeviceTensor(C, _F32)
        self.dbiases = DeviceTensor(C, _F32)
        if _wants_bf16(getattr(self, "prev", None)):
            _ck(_L().aeth_bn_bwd_twin_f32(self.inputs.ptr, dvalues.ptr, self.gamma.ptr, self.batch_mean.ptr,
                                          self.batch_invstd.ptr, self.dinputs.ptr, _twin(self.dinputs).ptr,
                                          self.dweights.ptr, self.dbiases.ptr, rows, C))
        else:
            _ck(_L().aeth_bn_bwd_f32(self.inputs.ptr, dvalues.ptr, self.gamma.ptr, self.batch_mean.ptr,
                                     self.batch_invstd.ptr, self.dinputs.ptr, self.dweights.ptr, self.dbiases.ptr,
                                     rows, C))
        return self.dinputs

    def get_parameters(self):
        return (self.gamma, self.beta, self.running_mean, self.running_var)

    def set_parameters(self, gamma, beta, running_mean, running_var):
        self.gamma = as_device(gamma, _F32).reshape(-1)
        self.beta = as_device(beta, _F32).reshape(-1)
        self.running_mean = as_device(running_mean, _F32)
        self.running_var = as_device(running_var, _F32)
        self.weights = self.gamma
        self.biases = self.beta


# ----------------------------------------------------------------------------------
# Flatten / SoftMax  (CNN_classes_cupy.py:528-563)
# ----------------------------------------------------------------------------------
class Flatten:
    def forward(self, inputs, training):
        inputs = as_device(inputs, _F32)
        self.inputs_shape = inputs.shape
        self.output = inputs.reshape(inputs.shape[0], -1)
        return self.output

    def backward(self, dvalues):
        self.dinputs = as_device(dvalues, _F32).reshape(self.inputs_shape)


class SoftMax:
    def forward(self, inputs, training=None):
        inputs = as_device(inputs, _F32)
        rows, K = inputs.shape
        self.output = DeviceTensor(inputs.shape, _F32)
        _ck(_L().aeth_softmax_f32(inputs.ptr, self.output.ptr, rows, K))
        return self.output

    def backward(self, dvalues):
        dvalues = as_device(dvalues, _F32)
        rows, K = dvalues.shape
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        _ck(_L().aeth_softmax_bwd_f32(self.output.ptr, dvalues.ptr, self.dinputs.ptr, rows, K))

    def predictions(self, outputs):
        # the loss kernel already produced the row argmax of these probabilities
        cached = getattr(outputs, "_cache", None)
        if cached is not None and "argmax" in cached:
            return cached["argmax"]
        return np.argmax(np.asarray(outputs), axis=1)


# ----------------------------------------------------------------------------------
# Loss  (CNN_classes_cupy.py:565-680)
# ----------------------------------------------------------------------------------
def _targets(y_true):
    """What the loss kernels take for `y_true`: ("index", int32 class indices) for a vector of labels or for
    one-hot rows, ("dense", float32 [S, K]) for any other 2-D array: soft or already smoothed targets, which the
    reference multiplies in as given (:622-626, :672-676)."""
    y = np.asarray(y_true)
    if y.ndim == 2:
        idx = np.argmax(y, axis=1)
        onehot = np.zeros(y.shape, dtype=y.dtype)
        onehot[np.arange(y.shape[0]), idx] = 1
        if np.array_equal(y, onehot):
            return "index", np.ascontiguousarray(idx, dtype=np.int32)
        return "dense", np.ascontiguousarray(y, dtype=_F32)
    return "index", np.ascontiguousarray(y, dtype=np.int32)


_label_cache = [None, None]     # (kind and bytes of the last target batch, its device copy)
_label_buffer = [None]          # while a step is being recorded: (kind, the buffer its kernels read the targets from)


def _device_targets(y_true):
    """(kind, targets on the device); the forward and backward pass of one step share the upload."""
    if _label_buffer[0] is not None:
        return _label_buffer[0]
    kind, y = _targets(y_true)
    key = (kind, y.shape, y.tobytes())
    if _label_cache[0] != key:
        _label_cache[0] = key
        _label_cache[1] = DeviceTensor.from_numpy(y, y.dtype)
    return kind, _label_cache[1]


def _for_targets(kind, index_fn, dense_fn):
    return getattr(_L(), index_fn if kind == "index" else dense_fn)


class Loss:
    def remember_trainable_layers(self, trainable_layers):
        self.trainable_layers = trainable_layers

    # ``calculate`` in two halves for Model.train_step: ``launch`` queues the loss kernel,
    # ``finish`` reads its result.  With backward and the optimizer queued in between, the
    # host never waits in the middle of a step.  Only for losses that offer
    # ``forward_launch``.  A regulariser's sums go the same way (``regularization_launch``
    # before the update is queued, so that they see the weights the reference's see;
    # ``regularization_finish`` after it).
    def can_defer(self):
        return hasattr(self, "forward_launch")

    def has_regularizer(self):
        return any(l.weight_regularizer_l1 > 0 or l.weight_regularizer_l2 > 0 or l.bias_regularizer_l1 > 0
                   or l.bias_regularizer_l2 > 0 for l in self.trainable_layers)

    def launch(self, output, y, *, training=True):
        return self.forward_launch(output, y, training)

    def finish(self, pending, *, include_regularization=False):
        sample_losses = self.forward_finish(pending)
        data_loss = np.mean(sample_losses)
        self.accumulated_sum += np.sum(sample_losses)
        self.accumulated_count += len(sample_losses)
        if not include_regularization:
            return data_loss
        return data_loss, self.regularization_loss()

    def calculate(self, output, y, *, include_regularization=False, training=True):
        sample_losses = self.forward(output, y, training)
        data_loss = np.mean(sample_losses)
        self.accumulated_sum += np.sum(sample_losses)
        self.accumulated_count += len(sample_losses)
        if not include_regularization:
            return data_loss
        return data_loss, self.regularization_loss()

    def calculate_accumulated(self, *, include_regularization=False):
        data_loss = self.accumulated_sum / self.accumulated_count
        if not include_regularization:
            return data_loss
        return data_loss, self.regularization_loss()

    def new_pass(self):
        self.accumulated_sum = 0
        self.accumulated_count = 0

    def regularization_launch(self):
        """Queues the sums of Loss.regularization_loss (CNN_classes_cupy.py:593-609), sum |x| (mode 0) or
        sum x^2 (1) per active coefficient in the reference's order, into one device buffer."""
        terms = []
        for layer in self.trainable_layers:
            if layer.weight_regularizer_l1 > 0:
                terms.append((layer.weight_regularizer_l1, layer.weights, 0))
            if layer.weight_regularizer_l2 > 0:
                terms.append((layer.weight_regularizer_l2, layer.weights, 1))
            if layer.bias_regularizer_l1 > 0:
                terms.append((layer.bias_regularizer_l1, layer.biases, 0))
            if layer.bias_regularizer_l2 > 0:
                terms.append((layer.bias_regularizer_l2, layer.biases, 1))
        if not terms:
            return None
        sums = DeviceTensor(len(terms), _F32)
        for i, (_, t, mode) in enumerate(terms):
            _ck(_L().aeth_reduce_f32(t.ptr, t.size, mode, sums.ptr + 4 * i))
        return [coef for coef, _, _ in terms], sums

    def regularization_finish(self, pending):
        """One read-back for all the sums; the weighted total is added up on the host in the reference's order."""
        regularization_loss = 0
        if pending is not None:
            coefs, sums = pending
            for coef, value in zip(coefs, sums.get()):
                regularization_loss += coef * float(value)
        return regularization_loss

    def regularization_loss(self):
        return self.regularization_finish(self.regularization_launch())


class Loss_CategoricalCrossEntropy(Loss):
    def __init__(self, label_smoothing=0.0):
        self.label_smoothing = label_smoothing

    def forward(self, y_pred, y_true, training=True):
        return self.forward_finish(self.forward_launch(y_pred, y_true, training))

    def forward_launch(self, y_pred, y_true, training=True):
        y_pred = as_device(y_pred, _F32)
        rows, K = y_pred.shape
        kind, labels = _device_targets(y_true)
        ls = self.label_smoothing if (self.label_smoothing > 0 and training) else 0.0
        # per-sample loss and row argmax side by side: one read-back for both
        buf = DeviceTensor(2 * rows, _F32)
        fn = _for_targets(kind, "aeth_cce_fwd_f32", "aeth_cce_fwd_dense_f32")
        _ck(fn(y_pred.ptr, labels.ptr, ls, buf.ptr, buf.ptr + 4 * rows, rows, K))
        return buf, rows, y_pred

    def forward_finish(self, pending):
        buf, rows, y_pred = pending
        host = buf.get()
        y_pred._cache = {"argmax": host[rows:].view(np.int32)}
        return host[:rows]

    def head_launch(self, logits, y_true, softmax, fused):
        """A training step's classifier head in one launch (Model.train_step): `softmax`'s output, this
        loss with the row argmax, and the gradient `fused` (the softmax / cross-entropy object) would work
        out in backward, which then finds it done.  The same operations in the same order as the three
        separate launches."""
        logits = as_device(logits, _F32)
        rows, K = logits.shape
        kind, labels = _device_targets(y_true)
        ls = self.label_smoothing if self.label_smoothing > 0 else 0.0
        probs = DeviceTensor(logits.shape, _F32)
        buf = DeviceTensor(2 * rows, _F32)
        dlogits = DeviceTensor(logits.shape, _F32)
        fn = _for_targets(kind, "aeth_softmax_cce_train_f32", "aeth_softmax_cce_train_dense_f32")
        _ck(fn(logits.ptr, labels.ptr, ls, probs.ptr, buf.ptr, buf.ptr + 4 * rows, dlogits.ptr, rows, K))
        softmax.output = probs
        fused.dinputs = dlogits
        fused._done_for = probs
        return buf, rows, probs

    def backward(self, dvalues, y_true):
        dvalues = as_device(dvalues, _F32)
        rows, K = dvalues.shape
        kind, labels = _device_targets(y_true)
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        fn = _for_targets(kind, "aeth_softmax_cce_bwd_f32", "aeth_softmax_cce_bwd_dense_f32")
        _ck(fn(dvalues.ptr, labels.ptr, self.label_smoothing, self.dinputs.ptr, rows, K))


class Activation_Softmax_Loss_CategoricalCrossEntropy():
    def __init__(self, label_smoothing=0.0):
        self.activation = SoftMax()
        self.loss = Loss_CategoricalCrossEntropy(label_smoothing)
        self.loss.new_pass()
        self.label_smoothing = label_smoothing

    def forward(self, inputs, y_true, training=True):
        self.activation.forward(inputs)
        self.output = self.activation.output
        return self.loss.calculate(self.output, y_true, training=training)

    def backward(self, dvalues, y_true, training=True):
        if getattr(self, "_done_for", None) is dvalues and dvalues is not None:
            self._done_for = None                        # the head kernel of this step has written dinputs
            return
        dvalues = as_device(dvalues, _F32)
        rows, K = dvalues.shape
        kind, labels = _device_targets(y_true)
        ls = self.label_smoothing if (self.label_smoothing > 0 and training) else 0.0
        self.dinputs = DeviceTensor(dvalues.shape, _F32)
        fn = _for_targets(kind, "aeth_softmax_cce_bwd_f32", "aeth_softmax_cce_bwd_dense_f32")
        _ck(fn(dvalues.ptr, labels.ptr, ls, self.dinputs.ptr, rows, K))


# ----------------------------------------------------------------------------------
# Optimizer_Adam  (CNN_classes_cupy.py:685-736)
# ----------------------------------------------------------------------------------
class Optimizer_Adam:
    def __init__(self, learning_rate=.001, decay=0., epsilon=1e-7, beta_1=0.9, beta_2=.999):
        self.learning_rate = learning_rate
        self.current_learning_rate = learning_rate
        self.decay = decay
        self.iterations = 0
        self.epsilon = epsilon
        self.beta_1 = beta_1
        self.beta_2 = beta_2
        self._pending = []

    def pre_update_parameters(self):
        if self.decay:
            self.current_learning_rate = self.learning_rate * (1. / (1. + self.decay * self.iterations))

    def update_parameters(self, layer):
        if not hasattr(layer, "weight_cache"):
            layer.weight_momentums = DeviceTensor.zeros(layer.weights.shape)
            layer.weight_cache = DeviceTensor.zeros(layer.weights.shape)
            layer.bias_momentums = DeviceTensor.zeros(layer.biases.shape)
            layer.bias_cache = DeviceTensor.zeros(layer.biases.shape)
        # The updates of all layers of a step go out as one launch: they are queued
        # here and issued by post_update_parameters (or when 32 tensors are waiting).
        self._pending.append((layer.weights, layer.dweights, layer.weight_momentums, layer.weight_cache))
        self._pending.append((layer.biases, layer.dbiases, layer.bias_momentums, layer.bias_cache))
        if len(self._pending) >= 32:
            self._flush()

    def _flush(self):
        import ctypes as C
        while self._pending:
            batch, self._pending = self._pending[:32], self._pending[32:]
            n = len(batch)
            arr = lambda k: (C.c_void_p * n)(*[t[k].ptr for t in batch])
            sizes = (C.c_int64 * n)(*[t[0].size for t in batch])
            for t in batch:
                if t[1].size != t[0].size:
                    raise ValueError("gradient shape %s does not match parameter shape %s" % (t[1].shape, t[0].shape))
            _ck(_L().aeth_adam_multi_f32(n, arr(0), arr(1), arr(2), arr(3), sizes, self.current_learning_rate,
                                         self.beta_1, self.beta_2, self.epsilon, self.iterations))
            for t in batch:
                t[0].touched()                               # the parameters changed in place

    def post_update_parameters(self):
        self._flush()
        self.iterations += 1

    # -- recorded steps: the step number lives on the device -----------------------------
    def device_state(self):
        """{iterations, beta_1^iterations, beta_2^iterations, lr} as 4 doubles on the device,
        brought in line with ``self.iterations`` whenever eager steps moved it."""
        if getattr(self, "_state", None) is None:
            self._state = DeviceTensor(4, np.float64)
            self._state_iterations = None
        if self._state_iterations != self.iterations:
            b1, b2 = float(np.float32(self.beta_1)), float(np.float32(self.beta_2))   # what the kernels receive
            self._state.set(np.array([self.iterations, b1 ** self.iterations, b2 ** self.iterations,
                                      self.current_learning_rate], dtype=np.float64))
            self._state_iterations = self.iterations
        return self._state

    def record_update(self, layers):
        """Queue one whole optimizer step (pre_update, every layer, post_update) in a form
        that can be replayed: learning rate and bias corrections come from device_state()."""
        import ctypes as C
        state = self._state
        self._recorded_params = [t for layer in layers for t in (layer.weights, layer.biases)]
        b1, b2 = float(np.float32(self.beta_1)), float(np.float32(self.beta_2))
        _ck(_L().aeth_adam_state_step(state.ptr, float(self.learning_rate), float(self.decay), b1, b2))
        batch = []
        for layer in layers:
            batch.append((layer.weights, layer.dweights, layer.weight_momentums, layer.weight_cache))
            batch.append((layer.biases, layer.dbiases, layer.bias_momentums, layer.bias_cache))
        while batch:
            part, batch = batch[:32], batch[32:]
            n = len(part)
            arr = lambda k: (C.c_void_p * n)(*[t[k].ptr for t in part])
            sizes = (C.c_int64 * n)(*[t[0].size for t in part])
            _ck(_L().aeth_adam_multi_dev_f32(n, arr(0), arr(1), arr(2), arr(3), sizes, self.beta_1, self.beta_2,
                                             self.epsilon, state.ptr))

    def replayed(self):
        """Host bookkeeping after a recorded step has run once more."""
        if self.decay:
            self.current_learning_rate = self.learning_rate * (1. / (1. + self.decay * self.iterations))
        self.iterations += 1
        self._state_iterations = self.iterations
        for t in getattr(self, "_recorded_params", ()):
            t.touched()
