"""Parameter files: the writer's cupy-style stream against the opcode stream of one of the
reference's own checkpoints (tests/golden/checkpoint_opcodes.json, made by
tests/golden/make_checkpoint_opcodes.py), and the loader on what the writer wrote."""
import hashlib
import io
import json
import os
import pickle
import pickletools
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "aether-ml_amd"))

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "checkpoint_opcodes.json")
# the reference's checkpoint: conv, batch norm, conv, batch norm, conv, batch norm, dense, dense
TUPLES = (2, 4, 2, 4, 2, 4, 2, 2)


def _params(golden, seed=0):
    r = np.random.RandomState(seed)
    arrays = [r.randn(*shape).astype({"f4": np.float32, "f8": np.float64}[dt]) for shape, dt in golden["arrays"]]
    out, i = [], 0
    for n in TUPLES:
        out.append(tuple(arrays[i:i + n]))
        i += n
    assert i == len(arrays)
    return out


def unframed_sha256(blob):
    """SHA-256 of a pickle stream with its FRAME opcodes left out (framing is where the
    writing pickler cut the stream, not content).  pickletools.genops executes nothing."""
    ops = [(op.name, pos) for op, _arg, pos in pickletools.genops(blob)]
    ends = [p for _, p in ops[1:]] + [len(blob)]
    h = hashlib.sha256()
    for (name, start), end in zip(ops, ends):
        if name != "FRAME":
            h.update(blob[start:end])
    return h.hexdigest()


def _ops(blob):
    ops = []
    for op, arg, _pos in pickletools.genops(io.BytesIO(blob)):
        if isinstance(arg, (bytes, bytearray)):
            arg = {"bytes": len(arg)}
        ops.append([op.name, arg])
    return ops


def test_cupy_style_files_have_the_opcode_stream_of_the_reference_checkpoints(tmp_path):
    from aether.model import write_parameters
    golden = json.load(open(GOLDEN))
    path = tmp_path / "params"
    write_parameters(_params(golden), str(path), cupy_arrays=True)
    ours = _ops(path.read_bytes())
    theirs = golden["ops"]
    # frames are a transport detail of the pickler that wrote the file (where it cuts the stream), not content
    strip = lambda ops: [o for o in ops if o[0] != "FRAME"]
    ours, theirs = strip(ours), strip(theirs)
    assert len(ours) == len(theirs)
    for i, (a, b) in enumerate(zip(ours, theirs)):
        assert a == b, "opcode %d: wrote %r, the reference's file has %r" % (i, a, b)


def test_the_loader_reads_both_kinds_of_file_and_nothing_else(tmp_path):
    from aether.model import write_parameters, _ArrayOnlyUnpickler
    golden = json.load(open(GOLDEN))
    params = _params(golden, 1)
    for cupy_arrays in (False, True):
        path = tmp_path / ("p%d" % cupy_arrays)
        write_parameters(params, str(path), cupy_arrays=cupy_arrays)
        got = _ArrayOnlyUnpickler(io.BytesIO(path.read_bytes())).load()
        assert [len(t) for t in got] == list(TUPLES)
        for t, u in zip(got, params):
            for a, b in zip(t, u):
                assert a.dtype == b.dtype and np.array_equal(a, b)
    # plain files are readable by pickle.load anywhere; cupy-style ones name cupy, which is not installed here
    assert isinstance(pickle.loads((tmp_path / "p0").read_bytes())[0][0], np.ndarray)
    with pytest.raises(ModuleNotFoundError):
        pickle.loads((tmp_path / "p1").read_bytes())
    # anything but arrays is refused
    evil = pickle.dumps([(os.getcwd,)])
    with pytest.raises(pickle.UnpicklingError):
        _ArrayOnlyUnpickler(io.BytesIO(evil)).load()


# ---- the reference's own checkpoints ------------------------------------------------------
DIGESTS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "checkpoint_digests.json")
WEIGHTS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model5_weights.npz")


def _model5_params():
    z = np.load(WEIGHTS)
    arrays = [z["a%02d" % i] for i in range(len(z.files))]
    out, i = [], 0
    for n in TUPLES:
        out.append(tuple(arrays[i:i + n]))
        i += n
    assert i == len(arrays)
    return arrays, out


def test_extracted_arrays_are_the_reference_checkpoints_arrays():
    """tests/golden/model5_weights.npz against the digests taken from the reference's file
    when the arrays were extracted, and the four checkpoints' common structure."""
    digests = json.load(open(DIGESTS))["models"]
    arrays, _ = _model5_params()
    want = digests["model5"]["arrays"]
    assert len(arrays) == len(want) == 22
    for a, (shape, dt, sha) in zip(arrays, want):
        assert list(a.shape) == shape and a.dtype.str[1:] == dt
        assert hashlib.sha256(a.tobytes()).hexdigest() == sha
    golden = json.load(open(GOLDEN))
    assert [[s, d] for s, d, _ in want] == golden["arrays"]
    for name in ("model2", "model3", "model4"):              # same network, other weights
        assert [[s, d] for s, d, _ in digests[name]["arrays"]] == golden["arrays"]
        assert digests[name]["unframed_sha256"] != digests["model5"]["unframed_sha256"]
    # conv / batch-norm tensors float32, running statistics (1,1,1,C), dense tensors float64
    assert [a.dtype.str[1:] for a in arrays] == ["f4"] * 18 + ["f8"] * 4
    assert arrays[4].shape == (1, 1, 1, 32) and arrays[18].shape == (1152, 256)


def test_writer_reproduces_the_reference_checkpoint_byte_for_byte(tmp_path):
    """write_parameters(cupy_arrays=True) on model5's arrays gives model5's pickle stream:
    every opcode and every payload byte outside the FRAME opcodes."""
    from aether.model import write_parameters, _ArrayOnlyUnpickler
    digests = json.load(open(DIGESTS))["models"]["model5"]
    arrays, params = _model5_params()
    path = tmp_path / "model5"
    write_parameters(params, str(path), cupy_arrays=True)
    blob = path.read_bytes()
    assert unframed_sha256(blob) == digests["unframed_sha256"]
    reference_file = "/root/reference/CNN/saved_models/model5"
    if os.path.exists(reference_file):                        # where the reference is at hand: the bytes themselves
        theirs = open(reference_file, "rb").read()
        assert unframed_sha256(theirs) == digests["unframed_sha256"]
        assert len(theirs) == digests["file_bytes"]
    # and the loader gives the arrays back, dtypes included
    got = _ArrayOnlyUnpickler(io.BytesIO(blob)).load()
    flat = [a for t in got for a in t]
    assert len(flat) == 22
    for a, b in zip(flat, arrays):
        assert a.dtype == b.dtype and a.shape == b.shape and np.array_equal(a, b)
