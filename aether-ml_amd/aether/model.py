"""Model orchestrator with the reference's method names, signatures, attribute
protocol and printed progress lines (CNN/models/CNN_model_cupy.py:5-392).  How the
layer chain is linked and how batches are cut is this module's own: one batch
iterator serves train / evaluate / predict, one step function serves eager and
recorded steps.  Batches are sliced on the host and uploaded once; every activation
then stays in HBM until the three printed scalars are read back.

Parameter files written by ``save_parameters`` hold plain NumPy arrays (a list
of per-layer tuples, the reference's structure).  ``load_parameters`` reads them
with a restricted unpickler that only rebuilds NumPy arrays; the wrapper the
reference's CuPy pickles use (``cupy._core.core.array``) is mapped to
``numpy.asarray`` so such a file loads without CuPy and without executing
anything else from it.
"""
import io
import os
import pickle
import warnings

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


def _batches(n_rows, batch_size):
    """Row ranges of one pass over `n_rows` samples: the whole set when no batch size is
    given, else consecutive batches with a shorter last one (CNN_model_cupy.py:81-92)."""
    if batch_size is None:
        yield slice(None)
        return
    for start in range(0, n_rows, batch_size):
        yield slice(start, start + batch_size)


def _rows(a, span):
    """`a[span]`, or `a` itself for the whole set (which may then be a DeviceTensor)."""
    return a if span == slice(None) else a[span]


def _progress(prefix, accuracy, loss, data_loss, regularization_loss, lr):
    """The reference's training line (CNN_model_cupy.py:127-133, :142-147), unbalanced
    bracket and doubled colon included."""
    return (f'{prefix}acc: {accuracy:.3f}, loss: {loss:.3f} (data_loss: {data_loss:.3f}, '
            f'reg_loss: {regularization_loss:.3f}, lr:: {lr}')


class Model:
    def __init__(self):
        self.layers = []
        self.softmax_classifier_output = None

    def add(self, layer):
        self.layers.append(layer)

    def set(self, *, loss=None, optimizer=None, accuracy=None):
        for name, value in (("loss", loss), ("optimizer", optimizer), ("accuracy", accuracy)):
            if value is not None:
                setattr(self, name, value)

    def finalize(self):
        """Links the chain (CNN_model_cupy.py:33-64): every layer gets .prev / .next, the
        first hangs on a Layer_Input, the last points at the loss; layers with `weights`
        are trainable; SoftMax + categorical cross-entropy get the fused backward."""
        self.input_layer = Layer_Input()
        chain = [self.input_layer] + self.layers + [self.loss]
        for before, layer, after in zip(chain, chain[1:], chain[2:]):
            layer.prev, layer.next = before, after
        self.output_layer_activation = self.layers[-1]
        self.trainable_layers = [layer for layer in self.layers if hasattr(layer, 'weights')]
        if self.loss is not None:
            self.loss.remember_trainable_layers(self.trainable_layers)
        fused = isinstance(self.layers[-1], SoftMax) and isinstance(self.loss, Loss_CategoricalCrossEntropy)
        if fused:
            self.softmax_classifier_output = \
                Activation_Softmax_Loss_CategoricalCrossEntropy(self.loss.label_smoothing)

    def train(self, X, y, *, epochs=1, batch_size=None, print_every=1, validation_data=None):
        self.accuracy.init(y)
        spans = list(_batches(len(X), batch_size))
        print("Training")
        for epoch in range(1, epochs + 1):
            print(f' epoch: {epoch}')
            self.loss.new_pass()
            self.accuracy.new_pass()
            # Steps are read one step late: the host queues step k + 1 while step k runs and takes step k's loss and
            # predictions afterwards; sums and printed lines are those of a loop that reads every step at once.
            waiting = []                                     # (step, function that reads its scalars)

            def report(step, loss, data_loss, regularization_loss, accuracy, lr):
                if step % print_every == 0 or step == len(spans) - 1:
                    print(_progress(f'epoch: {epoch}, ', accuracy, loss, data_loss, regularization_loss, lr))

            def drain(keep):
                while len(waiting) > keep:
                    k, finish = waiting.pop(0)
                    report(k, *finish())

            try:
                for step, rows in enumerate(spans):
                    batch_X, batch_y = _rows(X, rows), _rows(y, rows)
                    finish = self._recorded_step(batch_X, batch_y, later=True) if self.recording_active else None
                    if finish is None:
                        finish = self._eager_step(batch_X, batch_y, later=True)
                    if callable(finish):
                        waiting.append((step, finish))
                        drain(1)
                        continue
                    drain(0)                                 # results enter the sums in the order of the steps
                    report(step, *finish, self.optimizer.current_learning_rate)
                drain(0)
            finally:
                for _, finish in waiting:                    # (only after an exception: hand the pending copies back)
                    try:
                        finish()
                    except Exception:
                        pass
        # the summary and the validation pass come once, after the last epoch (:135-151)
        data_loss, regularization_loss = self.loss.calculate_accumulated(include_regularization=True)
        print(_progress(' training, ', self.accuracy.calculate_accumulated(), data_loss + regularization_loss,
                        data_loss, regularization_loss, self.optimizer.current_learning_rate))
        if validation_data is not None:
            self.evaluate(*validation_data, batch_size=batch_size)

    # -- recorded steps ------------------------------------------------------------------
    def record_steps(self, enabled=True):
        """Replay training steps from a recording instead of launching every kernel from
        Python (no counterpart in the reference).  The first step of a batch shape runs
        normally, the second is recorded as a HIP graph, later ones replay it: one host
        call per step.  Same kernels, same order, same results; the step number and the
        learning rate live on the device.  Dropout masks are still drawn on the host, in
        the layers' order from the reference's random stream, and copied into the buffers
        the recorded kernels read before every replay.  Regularisers are recorded: their
        sums and their gradient terms are kernels like the rest.  Falls back to normal
        steps for models the recording cannot express (anything but Adam with the fused
        softmax / cross-entropy output)."""
        self._record = bool(enabled)
        if not enabled:
            self._drop_recordings()
        elif not self._can_record():
            warnings.warn("record_steps: this model cannot be recorded (no Adam / fused softmax cross-entropy); "
                          "steps run eagerly", RuntimeWarning, stacklevel=2)

    @property
    def recording_active(self):
        """True when recording was asked for AND this model's steps can be recorded."""
        return bool(getattr(self, "_record", False)) and self._can_record()

    def _drop_recordings(self):
        from . import _lib
        for rec in getattr(self, "_recordings", {}).values():
            if rec.get("graph"):
                _lib.check(_lib.lib().aeth_graph_destroy(rec["graph"]))
        self._recordings = {}

    def _can_record(self):
        from .layers import Optimizer_Adam
        if self.softmax_classifier_output is None or not isinstance(self.optimizer, Optimizer_Adam):
            return False
        return self.loss.can_defer()

    def _recorded_step(self, batch_X, batch_y, later=False):
        """One step through a recording.  None: this step has to run normally (first step of a shape).  With
        `later` and a replay: a function that reads the step's scalars when called, instead of the scalars."""
        import ctypes as C
        from . import _lib, layers as L
        from .tensor import DeviceTensor
        kind, labels = L._targets(batch_y)
        key = (tuple(batch_X.shape), kind, labels.shape)
        recs = self.__dict__.setdefault("_recordings", {})
        rec = recs.get(key)
        if rec is None or not all(hasattr(l, "weight_cache") for l in self.trainable_layers):
            # first step of this shape, or no Adam state yet: a normal one (lazy initialisations,
            # workspace sizes)
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
            rec["labels"] = DeviceTensor(labels.shape, labels.dtype)
            self.optimizer.device_state()
            _lib.check(lib.aeth_graph_begin())
            L._label_buffer[0] = (kind, rec["labels"])
            L._recording[0] = True
            del L._recorded_masks[:]
            try:
                output, rec["pending"] = self._forward_and_loss(rec["x"], batch_y)
                rec["reg_pending"] = self.loss.regularization_launch()      # (before the update, as in train_step)
                rec["output"] = output
                self.backward(output, batch_y)
                self.optimizer.record_update(self.trainable_layers)
            finally:
                L._label_buffer[0] = None
                L._recording[0] = False
                rec["masks"] = list(L._recorded_masks)      # in the order the forward pass met the dropout layers
                del L._recorded_masks[:]
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
        for layer, buffer in rec["masks"]:                  # this step's dropout masks, drawn in the layers' order
            buffer.set(layer.host_mask(buffer.shape))
        _lib.check(lib.aeth_graph_launch(rec["graph"]))
        self.optimizer.replayed()
        if self.layers[-1].__dict__.get("output") is not rec["output"]:
            for obj, name, val in rec["bindings"]:
                setattr(obj, name, val)
        if not later:
            data_loss = self.loss.finish(rec["pending"])
            regularization_loss = self.loss.regularization_finish(rec.get("reg_pending"))
            predictions = self.output_layer_activation.predictions(rec["output"])
            accuracy = self.accuracy.calculate(predictions, batch_y)
            return data_loss + regularization_loss, data_loss, regularization_loss, accuracy
        return self._read_later(rec["pending"], rec.get("reg_pending"), batch_y)

    def _read_later(self, pending, reg, batch_y):
        """The step's scalars (per-sample losses with the predictions beside them, the regulariser's sums) are copied to
        the host behind what the step has queued and read when the caller asks for them, by which time the next step
        may be running (Model.train).  Returns the function that reads them: (loss, data loss, regularisation loss,
        accuracy, learning rate of the step)."""
        buf, rows, _ = pending
        loss_later = buf.get_later()
        reg_later = reg[1].get_later() if reg is not None else None
        lr = self.optimizer.current_learning_rate

        def finish():
            host = loss_later()
            sample_losses, predictions = host[:rows], host[rows:].view(np.int32)
            data_loss = np.mean(sample_losses)
            self.loss.accumulated_sum += np.sum(sample_losses)
            self.loss.accumulated_count += len(sample_losses)
            regularization_loss = 0
            if reg is not None:
                for coef, value in zip(reg[0], reg_later()):
                    regularization_loss += coef * float(value)
            accuracy = self.accuracy.calculate(predictions, batch_y)
            return data_loss + regularization_loss, data_loss, regularization_loss, accuracy, lr
        return finish

    def train_step(self, batch_X, batch_y):
        """One iteration of the loop body of ``train`` (CNN_model_cupy.py:107-126):
        forward, loss, accuracy, backward, Adam.  Returns (loss, data_loss,
        regularization_loss, accuracy)."""
        if self.recording_active:
            result = self._recorded_step(batch_X, batch_y)
            if result is not None:
                return result
        return self._eager_step(batch_X, batch_y)

    def _eager_step(self, batch_X, batch_y, later=False):
        """One step launched kernel by kernel.  With `later` (and a loss that can be queued): a function that reads the
        step's scalars when called, instead of the scalars."""
        # The loss kernel is queued here and read after backward and the update have been
        # queued too, so the device never idles while the host prepares the backward pass.
        # A regulariser's sums are queued here as well: they see the weights before the update,
        # as the reference's do (it works the loss out before backward, :113-115).
        reg_pending = None
        if self.loss.can_defer():
            output, pending = self._forward_and_loss(batch_X, batch_y)
            reg_pending = self.loss.regularization_launch()
        else:
            output, pending = self.forward(batch_X, training=True), None
        if pending is None:
            data_loss, regularization_loss = self.loss.calculate(output, batch_y, include_regularization=True,
                                                                 training=True)
        self.backward(output, batch_y)
        self.optimizer.pre_update_parameters()
        for layer in self.trainable_layers:
            self.optimizer.update_parameters(layer)
        self.optimizer.post_update_parameters()
        if later and pending is not None:
            return self._read_later(pending, reg_pending, batch_y)
        if pending is not None:
            data_loss = self.loss.finish(pending)
            regularization_loss = self.loss.regularization_finish(reg_pending)
        predictions = self.output_layer_activation.predictions(output)
        accuracy = self.accuracy.calculate(predictions, batch_y)
        return data_loss + regularization_loss, data_loss, regularization_loss, accuracy

    def _forward_and_loss(self, X, y):
        """The forward pass of a training step with the loss kernel queued behind it.  A SoftMax
        output under the fused softmax / cross-entropy object goes out as one launch with the loss,
        the predictions and the gradient of the logits (`AETHER_FUSE_HEAD=0` keeps them apart)."""
        head = self.layers[-1]
        if (self.softmax_classifier_output is None or not isinstance(head, SoftMax) or len(self.layers) < 2
                or not hasattr(self.loss, "head_launch") or os.environ.get("AETHER_FUSE_HEAD", "1") == "0"):
            output = self.forward(X, training=True)
            return output, self.loss.launch(output, y, training=True)
        self.input_layer.forward(X, True)
        for layer in self.layers[:-1]:
            layer.forward(layer.prev.output, True)
        logits = head.prev.output
        if len(getattr(logits, "shape", ())) != 2:
            head.forward(logits, True)
            return head.output, self.loss.launch(head.output, y, training=True)
        pending = self.loss.head_launch(logits, y, head, self.softmax_classifier_output)
        return head.output, pending

    def forward(self, X, training):
        """Every layer reads its predecessor's `.output` (CNN_model_cupy.py:153-163)."""
        self.input_layer.forward(X, training)
        for layer in self.layers:
            layer.forward(layer.prev.output, training)
        return self.layers[-1].output

    def backward(self, output, y):
        """Every layer reads its successor's `.dinputs` (CNN_model_cupy.py:165-193).  With the
        fused softmax / cross-entropy the last layer's dinputs come from the fused object."""
        if self.softmax_classifier_output is None:
            self.loss.backward(output, y)
            walk = self.layers
        else:
            self.softmax_classifier_output.backward(output, y, training=True)
            self.layers[-1].dinputs = self.softmax_classifier_output.dinputs
            walk = self.layers[:-1]
        for layer in reversed(walk):
            layer.backward(layer.next.dinputs)

    def backward_debug(self, X, y):
        """One training forward and backward pass that prints every layer's output shape, then every
        layer's gradient shapes (CNN_model_cupy.py:195-229); the reference's scripts call it on one
        sample before training.  No loss is computed and no parameter changes."""
        print("Forward pass:")
        self.input_layer.forward(X, True)
        for i, layer in enumerate(self.layers):
            layer.forward(layer.prev.output, True)
            print(f"Layer {i} ({layer.__class__.__name__}) output: {tuple(layer.output.shape)}")
        print("\nBackward pass:")
        self.backward(self.layers[-1].output, y)
        fused = self.softmax_classifier_output is not None
        walk = self.layers[:-1] if fused else self.layers
        for i, layer in enumerate(reversed(walk)):
            print(f"Layer {-i - (2 if fused else 1)} ({layer.__class__.__name__}) dinputs: {tuple(layer.dinputs.shape)}")
            for name in ("dweights", "dbiases"):
                if hasattr(layer, name):
                    print(f"             {name}: {tuple(getattr(layer, name).shape)}")

    def evaluate(self, X_val, y_val, *, batch_size=None):
        self.loss.new_pass()
        self.accuracy.new_pass()
        for rows in _batches(len(X_val), batch_size):
            batch_y = _rows(y_val, rows)
            output = self.forward(_rows(X_val, rows), training=False)
            self.loss.calculate(output, batch_y, training=False)
            self.accuracy.calculate(self.output_layer_activation.predictions(output), batch_y)
        validation_loss = self.loss.calculate_accumulated()
        validation_accuracy = self.accuracy.calculate_accumulated()
        print(f'Valdiation, acc: {validation_accuracy:.3f}, loss: {validation_loss:.3f}')

    def predict(self, X, *, batch_size=None):
        parts = [np.asarray(self.forward(_rows(X, rows), training=False)) for rows in _batches(len(X), batch_size)]
        return np.vstack(parts)

    def get_parameters(self):
        return [layer.get_parameters() for layer in self.trainable_layers]

    def set_parameters(self, parameters):
        for layer, parameter_set in zip(self.trainable_layers, parameters):
            layer.set_parameters(*parameter_set)

    def save_parameters(self, path, cupy_arrays=False):
        """`cupy_arrays`: the stream of the reference's CuPy checkpoints, dtypes included: its dense layers hold
        float64 parameters (`cp.random.randn`, CNN_classes_cupy.py:320-322; `CNN/saved_models/model5` stores them
        as f8), so the float32 dense parameters of this build are widened (exactly) on the way out."""
        from .layers import Layer_Dense
        params = []
        for layer in self.trainable_layers:
            tup = tuple(np.asarray(a) for a in layer.get_parameters())
            if cupy_arrays and isinstance(layer, Layer_Dense):
                tup = tuple(a.astype(np.float64) for a in tup)
            params.append(tup)
        write_parameters(params, path, cupy_arrays)

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


class Accuracy:
    """Running share of correct predictions (CNN_model_cupy.py:344-366): subclasses say
    what "correct" means through ``compare``."""

    def new_pass(self):
        self.accumulated_sum = 0
        self.accumulated_count = 0

    def calculate(self, predictions, y):
        hits = self.compare(predictions, y)
        self.accumulated_sum += np.sum(hits)
        self.accumulated_count += len(hits)
        return np.mean(hits)

    def calculate_accumulated(self):
        return self.accumulated_sum / self.accumulated_count


class Accuracy_Regression(Accuracy):
    """A prediction counts as correct within std(y) / 250 of the target (CNN_model_cupy.py:367-378)."""

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
        labels = np.argmax(y, axis=1) if y.ndim == 2 else y
        return np.asarray(predictions) == labels


class Layer_Input:
    def forward(self, inputs, training):
        self.output = inputs
