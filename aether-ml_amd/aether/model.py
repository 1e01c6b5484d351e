"""Model orchestrator with the reference's method names and behaviour
(CNN/models/CNN_model_cupy.py:5-392): layer chain, batching loop, loss/accuracy
bookkeeping and the printed progress lines.  Batches are sliced on the host and
uploaded once; every activation then stays in HBM until the three printed
scalars are read back.

Parameter files written by ``save_parameters`` hold plain NumPy arrays (a list
of per-layer tuples, the reference's structure).  ``load_parameters`` reads them
with a restricted unpickler that only rebuilds NumPy arrays; the wrapper the
reference's CuPy pickles use (``cupy._core.core.array``) is mapped to
``numpy.asarray`` so such a file loads without CuPy and without executing
anything else from it.
"""
import io
import pickle

import numpy as np

from .layers import (Activation_Softmax_Loss_CategoricalCrossEntropy, Loss_CategoricalCrossEntropy, SoftMax)


class _ArrayOnlyUnpickler(pickle.Unpickler):
    _ALLOWED = {
        ("numpy.core.multiarray", "_reconstruct"),
        ("numpy._core.multiarray", "_reconstruct"),
        ("numpy", "ndarray"),
        ("numpy", "dtype"),
        ("numpy.core.multiarray", "scalar"),
        ("numpy._core.multiarray", "scalar"),
    }

    def find_class(self, module, name):
        if (module, name) in self._ALLOWED:
            return super().find_class(module, name)
        if module.startswith("cupy") and name == "array":
            return np.asarray
        raise pickle.UnpicklingError("parameter files may only contain NumPy arrays (found %s.%s)" % (module, name))


def _cupy_array(a):
    """Stands for `cupy._core.core.array` in parameter files written for the reference's CuPy model."""
    raise RuntimeError("a marker for the pickler, never called")


class _CupyWrapped:
    """Pickles as `cupy._core.core.array(ndarray)`, which is how the reference's CuPy model's
    `save_parameters` stores an array (CNN/models/CNN_model_cupy.py:320-323 pickles
    `get_parameters()`, a list of tuples of cupy arrays)."""

    def __init__(self, a):
        self.a = a

    def __reduce__(self):
        return (_cupy_array, (self.a,))


class _CupyStylePickler(pickle._Pickler):
    """The pure-Python pickler with one global written under another name: cupy is not importable
    here, and the stock pickler refuses a global it cannot import."""

    def save_global(self, obj, name=None):
        if obj is _cupy_array:
            self.save("cupy._core.core")
            self.save("array")
            self.write(pickle.STACK_GLOBAL)
            self.memoize(obj)
            return
        super().save_global(obj, name)

    dispatch = dict(pickle._Pickler.dispatch)
    dispatch[type(_cupy_array)] = save_global


def write_parameters(params, path, cupy_arrays=False):
    """Writes a list of per-layer tuples of host arrays as the reference's parameter files are
    written: pickle protocol 4 of the list.  With `cupy_arrays` every array is stored as
    `cupy._core.core.array(ndarray)`, so that the reference's CuPy model can `load_parameters`
    the file (its checkpoints under CNN/saved_models have exactly this stream); without, as plain
    NumPy arrays, which `pickle.load` reads anywhere."""
    host = [tuple(np.ascontiguousarray(a) for a in tup) for tup in params]
    with open(path, 'wb') as f:
        if cupy_arrays:
            _CupyStylePickler(f, protocol=4).dump([tuple(_CupyWrapped(a) for a in tup) for tup in host])
        else:
            pickle.dump(host, f, protocol=4)


class Model:
    def __init__(self):
        self.layers = []
        self.softmax_classifier_output = None

    def add(self, layer):
        self.layers.append(layer)

    def set(self, *, loss=None, optimizer=None, accuracy=None):
        if loss is not None:
            self.loss = loss
        if optimizer is not None:
            self.optimizer = optimizer
        if accuracy is not None:
            self.accuracy = accuracy

    def finalize(self):
        self.input_layer = Layer_Input()
        layer_count = len(self.layers)
        self.trainable_layers = []
        for i in range(layer_count):
            if i == 0:
                self.layers[i].prev = self.input_layer
                self.layers[i].next = self.layers[i + 1]
            elif i < layer_count - 1:
                self.layers[i].prev = self.layers[i - 1]
                self.layers[i].next = self.layers[i + 1]
            else:
                self.layers[i].prev = self.layers[i - 1]
                self.layers[i].next = self.loss
                self.output_layer_activation = self.layers[i]
            if hasattr(self.layers[i], 'weights'):
                self.trainable_layers.append(self.layers[i])
        if self.loss is not None:
            self.loss.remember_trainable_layers(self.trainable_layers)
        if isinstance(self.layers[-1], SoftMax) and isinstance(self.loss, Loss_CategoricalCrossEntropy):
            self.softmax_classifier_output = \
                Activation_Softmax_Loss_CategoricalCrossEntropy(self.loss.label_smoothing)

    def train(self, X, y, *, epochs=1, batch_size=None, print_every=1, validation_data=None):
        self.accuracy.init(y)
        train_steps = 1
        if validation_data is not None:
            X_val, y_val = validation_data
        if batch_size is not None:
            train_steps = len(X) // batch_size
            if train_steps * batch_size < len(X):
                train_steps += 1
        print("Training")
        for epoch in range(1, epochs + 1):
            print(f' epoch: {epoch}')
            self.loss.new_pass()
            self.accuracy.new_pass()
            for step in range(train_steps):
                if batch_size is None:
                    batch_X = X
                    batch_y = y
                else:
                    batch_X = X[step * batch_size:(step + 1) * batch_size]
                    batch_y = y[step * batch_size:(step + 1) * batch_size]
                loss, data_loss, regularization_loss, accuracy = self.train_step(batch_X, batch_y)
                if not step % print_every or step == train_steps - 1:
                    print(f'epoch: {epoch}, ' +
                          f'acc: {accuracy:.3f}, ' +
                          f'loss: {loss:.3f} (' +
                          f'data_loss: {data_loss:.3f}, ' +
                          f'reg_loss: {regularization_loss:.3f}, ' +
                          f'lr:: {self.optimizer.current_learning_rate}')
        epoch_data_loss, epoch_regularization_loss = \
            self.loss.calculate_accumulated(include_regularization=True)
        epoch_loss = epoch_data_loss + epoch_regularization_loss
        epoch_accuracy = self.accuracy.calculate_accumulated()
        print(f' training, ' +
              f'acc: {epoch_accuracy:.3f}, ' +
              f'loss: {epoch_loss:.3f} (' +
              f'data_loss: {epoch_data_loss:.3f}, ' +
              f'reg_loss: {epoch_regularization_loss:.3f}, ' +
              f'lr:: {self.optimizer.current_learning_rate}')
        if validation_data is not None:
            self.evaluate(*validation_data, batch_size=batch_size)

    # -- recorded steps ------------------------------------------------------------------
    def record_steps(self, enabled=True):
        """Replay training steps from a recording instead of launching every kernel from
        Python (no counterpart in the reference).  The first step of a batch shape runs
        normally, the second is recorded as a HIP graph, later ones replay it: one host
        call per step.  Same kernels, same order, same results; the step number and the
        learning rate live on the device.  Falls back to normal steps for models the
        recording cannot express (dropout masks drawn on the host, active regularisers,
        anything but Adam with the fused softmax / cross-entropy output)."""
        self._record = bool(enabled)
        if not enabled:
            self._drop_recordings()

    def _drop_recordings(self):
        from . import _lib
        for rec in getattr(self, "_recordings", {}).values():
            if rec.get("graph"):
                _lib.check(_lib.lib().aeth_graph_destroy(rec["graph"]))
        self._recordings = {}

    def _can_record(self):
        from .layers import Layer_Dropout, Layer_Dropout_Spatial, Optimizer_Adam
        if self.softmax_classifier_output is None or not isinstance(self.optimizer, Optimizer_Adam):
            return False
        if not self.loss.can_defer():
            return False
        if any(isinstance(layer, (Layer_Dropout, Layer_Dropout_Spatial)) for layer in self.layers):
            return False                                 # their masks are drawn and uploaded by the host every step
        return all(hasattr(l, "weight_cache") for l in self.trainable_layers)     # Adam state exists

    def _recorded_step(self, batch_X, batch_y):
        import ctypes as C
        from . import _lib, layers as L
        from .tensor import DeviceTensor
        labels = L._sparse_labels(batch_y)
        key = (tuple(batch_X.shape), labels.shape[0])
        recs = self.__dict__.setdefault("_recordings", {})
        rec = recs.get(key)
        if rec is None:
            # first step of this shape: a normal one (lazy initialisations, workspace sizes)
            recs[key] = {"graph": None}
            return None
        lib = _lib.lib()
        # a recording reads and writes the parameter buffers it was made with: parameters set
        # anew since then (set_parameters, load_parameters) make it stale
        params = [(id(l), l.weights.ptr, l.biases.ptr) for l in self.trainable_layers]
        if rec["graph"] is not None and rec.get("params") != params:
            _lib.check(lib.aeth_graph_destroy(rec["graph"]))
            recs[key] = rec = {"graph": None}
        if rec["graph"] is None:
            rec["x"] = DeviceTensor(batch_X.shape, np.float32)
            rec["labels"] = DeviceTensor(labels.shape, np.int32)
            self.optimizer.device_state()
            _lib.check(lib.aeth_graph_begin())
            L._label_buffer[0] = rec["labels"]
            try:
                output = self.forward(rec["x"], training=True)
                rec["pending"] = self.loss.launch(output, batch_y, training=True)
                rec["output"] = output
                self.backward(output, batch_y)
                self.optimizer.record_update(self.trainable_layers)
            finally:
                L._label_buffer[0] = None
                handle = C.c_void_p()
                rc = lib.aeth_graph_end(C.byref(handle))
            _lib.check(rc)
            rec["graph"] = handle
            rec["params"] = params
            # what the layers point at after this step (output, dinputs, dweights, ...):
            # replays fill the same buffers, so the attributes are put back after steps
            # that ran in between (an evaluation, a step of another shape)
            holders = list(self.layers) + [self.softmax_classifier_output, self.softmax_classifier_output.activation,
                                           self.loss]
            rec["bindings"] = [(obj, name, val) for obj in holders for name, val in vars(obj).items()
                               if isinstance(val, DeviceTensor)]
        # feed the recording and replay it
        self.optimizer.device_state()
        if isinstance(batch_X, DeviceTensor):
            _lib.check(lib.aeth_memcpy_d2d(rec["x"].ptr, batch_X.ptr, rec["x"].nbytes))
        else:
            rec["x"].set(np.asarray(batch_X, dtype=np.float32))
        rec["labels"].set(labels)
        _lib.check(lib.aeth_graph_launch(rec["graph"]))
        self.optimizer.replayed()
        if self.layers[-1].__dict__.get("output") is not rec["output"]:
            for obj, name, val in rec["bindings"]:
                setattr(obj, name, val)
        data_loss, regularization_loss = self.loss.finish(rec["pending"], include_regularization=True)
        loss = data_loss + regularization_loss
        predictions = self.output_layer_activation.predictions(rec["output"])
        accuracy = self.accuracy.calculate(predictions, batch_y)
        return loss, data_loss, regularization_loss, accuracy

    def train_step(self, batch_X, batch_y):
        """One iteration of the loop body of ``train`` (CNN_model_cupy.py:107-126):
        forward, loss, accuracy, backward, Adam.  Returns (loss, data_loss,
        regularization_loss, accuracy)."""
        if getattr(self, "_record", False) and self._can_record():
            result = self._recorded_step(batch_X, batch_y)
            if result is not None:
                return result
        output = self.forward(batch_X, training=True)
        # The loss kernel is queued here and read after backward and the update have been
        # queued too, so the device never idles while the host prepares the backward pass.
        defer = self.loss.can_defer()
        if defer:
            pending = self.loss.launch(output, batch_y, training=True)
        else:
            data_loss, regularization_loss = self.loss.calculate(output, batch_y, include_regularization=True,
                                                                 training=True)
        self.backward(output, batch_y)
        self.optimizer.pre_update_parameters()
        for layer in self.trainable_layers:
            self.optimizer.update_parameters(layer)
        self.optimizer.post_update_parameters()
        if defer:
            data_loss, regularization_loss = self.loss.finish(pending, include_regularization=True)
        loss = data_loss + regularization_loss
        predictions = self.output_layer_activation.predictions(output)
        accuracy = self.accuracy.calculate(predictions, batch_y)
        return loss, data_loss, regularization_loss, accuracy

    def forward(self, X, training):
        self.input_layer.forward(X, training)
        for layer in self.layers:
            layer.forward(layer.prev.output, training)
        return layer.output

    def backward(self, output, y):
        if self.softmax_classifier_output is not None:
            self.softmax_classifier_output.backward(output, y, training=True)
            self.layers[-1].dinputs = self.softmax_classifier_output.dinputs
            for layer in reversed(self.layers[:-1]):
                layer.backward(layer.next.dinputs)
            return
        self.loss.backward(output, y)
        for layer in reversed(self.layers):
            layer.backward(layer.next.dinputs)

    def backward_debug(self, X, y):
        out = X
        print("Forward pass:")
        for i, layer in enumerate(self.layers):
            layer.forward(out, training=True)
            out = layer.output
            print(f"Layer {i} ({layer.__class__.__name__}) output: {out.shape}")
        print("\nBackward pass:")
        if self.softmax_classifier_output is not None:
            self.softmax_classifier_output.backward(out, y)
            self.layers[-1].dinputs = self.softmax_classifier_output.dinputs
            chain = list(enumerate(reversed(self.layers[:-1])))
            first = -2
        else:
            self.loss.backward(out, y)
            chain = list(enumerate(reversed(self.layers)))
            first = -1
        for i, layer in chain:
            layer.backward(layer.next.dinputs)
            print(f"Layer {first - i} ({layer.__class__.__name__}) dinputs: {layer.dinputs.shape}")
            if hasattr(layer, 'dweights'):
                print(f"             dweights: {layer.dweights.shape}")
            if hasattr(layer, 'dbiases'):
                print(f"             dbiases: {layer.dbiases.shape}")

    def evaluate(self, X_val, y_val, *, batch_size=None):
        validation_steps = 1
        if batch_size is not None:
            validation_steps = len(X_val) // batch_size
            if validation_steps * batch_size < len(X_val):
                validation_steps += 1
        self.loss.new_pass()
        self.accuracy.new_pass()
        for step in range(validation_steps):
            if batch_size is None:
                batch_X = X_val
                batch_y = y_val
            else:
                batch_X = X_val[step * batch_size:(step + 1) * batch_size]
                batch_y = y_val[step * batch_size:(step + 1) * batch_size]
            output = self.forward(batch_X, training=False)
            self.loss.calculate(output, batch_y, training=False)
            predictions = self.output_layer_activation.predictions(output)
            self.accuracy.calculate(predictions, batch_y)
        validation_loss = self.loss.calculate_accumulated()
        validation_accuracy = self.accuracy.calculate_accumulated()
        print(f'Valdiation, ' +
              f'acc: {validation_accuracy:.3f}, ' +
              f'loss: {validation_loss:.3f}')

    def get_parameters(self):
        parameters = []
        for layer in self.trainable_layers:
            parameters.append(layer.get_parameters())
        return parameters

    def set_parameters(self, parameters):
        for parameter_set, layer in zip(parameters, self.trainable_layers):
            layer.set_parameters(*parameter_set)

    def save_parameters(self, path, cupy_arrays=False):
        write_parameters([tuple(np.asarray(a) for a in tup) for tup in self.get_parameters()], path, cupy_arrays)

    def load_parameters(self, path):
        with open(path, 'rb') as f:
            self.set_parameters(_ArrayOnlyUnpickler(io.BytesIO(f.read())).load())

    def save(self, path):
        raise NotImplementedError(
            "whole-model pickles are not supported (device buffers cannot be pickled); use save_parameters")

    @staticmethod
    def load(path):
        raise NotImplementedError(
            "whole-model pickles are not supported (device buffers cannot be pickled); use load_parameters")

    def predict(self, X, *, batch_size=None):
        prediction_steps = 1
        if batch_size is not None:
            prediction_steps = len(X) // batch_size
            if prediction_steps * batch_size < len(X):
                prediction_steps += 1
        output = []
        for step in range(prediction_steps):
            if batch_size is None:
                batch_X = X
            else:
                batch_X = X[step * batch_size:(step + 1) * batch_size]
            batch_output = self.forward(batch_X, training=False)
            output.append(np.asarray(batch_output))
        return np.vstack(output)


class Accuracy:
    def calculate(self, predictions, y):
        comparisons = self.compare(predictions, y)
        accuracy = np.mean(comparisons)
        self.accumulated_sum += np.sum(comparisons)
        self.accumulated_count += len(comparisons)
        return accuracy

    def calculate_accumulated(self):
        accuracy = self.accumulated_sum / self.accumulated_count
        return accuracy

    def new_pass(self):
        self.accumulated_sum = 0
        self.accumulated_count = 0


class Accuracy_Regression(Accuracy):
    def __init__(self):
        self.precision = None

    def init(self, y, reinit=False):
        if self.precision is None or reinit:
            self.precision = np.std(np.asarray(y)) / 250

    def compare(self, predictions, y):
        return np.absolute(np.asarray(predictions) - np.asarray(y)) < self.precision


class Accuracy_Categorical(Accuracy):
    def init(self, y):
        pass

    def compare(self, predictions, y):
        y = np.asarray(y)
        if len(y.shape) == 2:
            y = np.argmax(y, axis=1)
        return np.asarray(predictions) == y


class Layer_Input:
    def forward(self, inputs, training):
        self.output = inputs
