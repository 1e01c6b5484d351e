"""Extracts the arrays of the reference's parameter checkpoints without unpickling them.

    python tests/golden/make_checkpoint_weights.py /root/reference/CNN/saved_models

The files (CNN/saved_models/model2..5, written by CNN/models/CNN_model_cupy.py:320-323) are
walked with pickletools.genops, which decodes the opcode stream and executes nothing from it.
An ndarray appears in the stream as  MARK, 1, (shape), dtype, fortran-flag, BINBYTES data, BUILD;
the shape is the run of small integers, the item size follows from len(data) / prod(shape), and
the only dtype strings the streams name are 'f4' and 'f8' (checked).  Written next to this script:

  model5_weights.npz       every array of model5 as a00..a21, in stream order (the F-MNIST
                           network of CNN/architectures/CNN_test2_cupy.py:31-59: conv, batch
                           norm, conv, batch norm, conv, batch norm, dense, dense)
  checkpoint_digests.json  for model2..5: shapes, dtypes and the SHA-256 of every array's bytes,
                           and the SHA-256 of the whole stream with the FRAME opcodes left out
                           (framing says where the writing pickler cut the stream; it is not content)
"""
import hashlib
import json
import os
import pickletools
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
BYTES_OPS = ("BINBYTES", "SHORT_BINBYTES", "BINBYTES8")


def walk(path):
    """(opcode name, argument, start, end) for every opcode of the file."""
    blob = open(path, "rb").read()
    ops = [(op.name, arg, pos) for op, arg, pos in pickletools.genops(blob)]
    ends = [p for _, _, p in ops[1:]] + [len(blob)]
    return blob, [(n, a, p, e) for (n, a, p), e in zip(ops, ends)]


def unframed_digest(blob, ops):
    h = hashlib.sha256()
    for name, _arg, start, end in ops:
        if name != "FRAME":
            h.update(blob[start:end])
    return h.hexdigest()


def arrays_of(ops):
    names = {a for n, a, _, _ in ops if n == "SHORT_BINUNICODE"}
    dtypes = {a for a in names if len(a) == 2 and a[0] in "fiub" and a[1].isdigit()}
    assert dtypes <= {"f4", "f8"}, dtypes
    out = []
    i = 0
    while i + 2 < len(ops):
        if ops[i][0] == "MARK" and ops[i + 1][:2] == ("BININT1", 1) and \
                (ops[i + 2][0] == "MARK" or ops[i + 2][0].startswith("BININT")):
            j = i + 3 if ops[i + 2][0] == "MARK" else i + 2
            shape = []
            while ops[j][0].startswith("BININT"):
                shape.append(ops[j][1])
                j += 1
            k = j
            while ops[k][0] not in BYTES_OPS:
                k += 1
            fortran = [n for n, _, _, _ in ops[j:k] if n in ("NEWTRUE", "NEWFALSE")][-1] == "NEWTRUE"
            assert not fortran
            data = ops[k][1]
            n = int(np.prod(shape)) if shape else 1
            item = len(data) // n
            assert item * n == len(data) and item in (4, 8)
            out.append(np.frombuffer(data, dtype="<f%d" % item).reshape(shape).copy())
            i = k
        i += 1
    return out


def main(folder):
    digests = {}
    for name in ("model2", "model3", "model4", "model5"):
        blob, ops = walk(os.path.join(folder, name))
        arrays = arrays_of(ops)
        digests[name] = {
            "file_bytes": len(blob),
            "unframed_sha256": unframed_digest(blob, ops),
            "arrays": [[list(a.shape), a.dtype.str[1:], hashlib.sha256(a.tobytes()).hexdigest()] for a in arrays],
        }
        print(name, len(arrays), "arrays", [tuple(a.shape) for a in arrays][:3], "...")
        if name == "model5":
            np.savez(os.path.join(HERE, "model5_weights.npz"), **{"a%02d" % i: a for i, a in enumerate(arrays)})
    with open(os.path.join(HERE, "checkpoint_digests.json"), "w") as f:
        json.dump({"source": "CNN/saved_models of the reference", "models": digests}, f, indent=1)


if __name__ == "__main__":
    main(sys.argv[1])
