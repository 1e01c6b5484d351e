"""Writes checkpoint_opcodes.json: the pickle opcode stream of one of the reference's parameter
checkpoints (CNN/saved_models/model5), with every bytes argument replaced by its length, plus the
shapes and dtypes of the arrays in it.  The file is parsed with pickletools.genops, which walks
the opcodes and executes nothing from the file; no array data is kept.

    python tests/golden/make_checkpoint_opcodes.py /root/reference/CNN/saved_models/model5
"""
import json
import os
import pickletools
import sys


def main(path):
    ops = []
    with open(path, "rb") as f:
        for op, arg, _pos in pickletools.genops(f):
            if isinstance(arg, (bytes, bytearray)):
                arg = {"bytes": len(arg)}
            ops.append([op.name, arg])
    # An ndarray's state is BUILD(version = 1, shape, dtype, fortran, data): its shape is the run of small
    # integers after the "MARK, 1" that opens the state, its item size the length of the data that follows
    # divided by the number of elements (the dtype object itself is memoized after its first use).
    arrays = []
    i = 0
    while i + 2 < len(ops):
        if ops[i][0] == "MARK" and ops[i + 1] == ["BININT1", 1] and (ops[i + 2][0] == "MARK" or ops[i + 2][0].startswith("BININT")):
            j = i + 3 if ops[i + 2][0] == "MARK" else i + 2
            shape = []
            while ops[j][0].startswith("BININT"):
                shape.append(ops[j][1])
                j += 1
            k = j
            while not (ops[k][0] in ("BINBYTES", "SHORT_BINBYTES", "BINBYTES8") and isinstance(ops[k][1], dict)):
                k += 1
            n = 1
            for d in shape:
                n *= d
            arrays.append([shape, "f%d" % (ops[k][1]["bytes"] // n)])
            i = k
        i += 1
    out = {"source": "CNN/saved_models/model5 of the reference", "protocol": ops[0][1], "ops": ops, "arrays": arrays}
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "checkpoint_opcodes.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(len(ops), "opcodes,", len(arrays), "arrays")
    for a in arrays:
        print(a)


if __name__ == "__main__":
    main(sys.argv[1])
