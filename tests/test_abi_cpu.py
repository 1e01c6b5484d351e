"""CPU-side checks of the C ABI: the library loads, exports every function the
header declares, the ctypes table matches the header, and calls made before
aeth_init fail with a status code instead of touching a GPU."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aether_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = re.findall(r"\b(?:int|const char\*)\s+(aeth_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S)
    return {name: [a.strip() for a in args.split(",")] if args.strip() not in ("", "void") else []
            for name, args in decls}


@pytest.fixture(scope="module")
def lib():
    from aether import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return _lib.load()


def test_header_declares_the_hot_path():
    d = _declared()
    for name in ("aeth_conv_fprop_f32", "aeth_conv_dgrad_f32", "aeth_conv_wgrad_f32",
                 "aeth_conv_fprop_bf16", "aeth_conv_dgrad_bf16", "aeth_conv_wgrad_bf16",
                 "aeth_dense_fprop_f32", "aeth_dense_dgrad_f32", "aeth_dense_wgrad_f32",
                 "aeth_init", "aeth_malloc", "aeth_last_error"):
        assert name in d
    assert len(d) >= 40


def test_library_exports_every_declared_symbol(lib):
    for name in _declared():
        assert hasattr(lib, name), name


def test_ctypes_table_matches_header(lib):
    from aether import _lib
    d = _declared()
    d.pop("aeth_last_error")
    assert set(d) == set(_lib.SIGNATURES)
    for name, args in d.items():
        assert len(args) == len(_lib.SIGNATURES[name]), name
        for decl, ct in zip(args, _lib.SIGNATURES[name]):
            if "*" in decl:
                assert ct in (ctypes.c_void_p, ctypes.c_char_p) or hasattr(ct, "contents"), (name, decl)
            elif decl.startswith("float"):
                assert ct is ctypes.c_float, (name, decl)
            elif decl.startswith("double"):
                assert ct is ctypes.c_double, (name, decl)
            elif decl.startswith("int64_t"):
                assert ct is ctypes.c_int64, (name, decl)
            else:
                assert decl.startswith("int") and ct is ctypes.c_int, (name, decl)


def test_no_torch_or_python_types_in_the_abi():
    text = open(HEADER).read()
    assert "torch" not in text.lower() and "PyObject" not in text and "#include <hip" not in text
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(ROOT, "aether-ml_amd", "aether", "lib",
                                                                    "libaether_hip.so")],
                         capture_output=True, text=True).stdout
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    assert set(_declared()) <= exported


def test_calls_before_init_report_state_error(lib):
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present: the context may already be initialised by other tests")
    assert lib.aeth_sync() == -4
    assert b"aeth_init" in lib.aeth_last_error()
    p = ctypes.c_void_p()
    assert lib.aeth_malloc(ctypes.byref(p), 16) == -4
    assert lib.aeth_conv_fprop_f32(None, None, None, None, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0) == -4
    # without a GPU aeth_init fails with a HIP error and a message, it does not abort
    assert lib.aeth_init(0) == -2
    assert b"aeth_init" in lib.aeth_last_error()


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "aether-ml_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)


def test_targets_are_indices_or_dense_rows():
    """Host logic of the loss: labels and one-hot rows become class indices; any other 2-D array (soft or
    already smoothed targets, which the reference uses as given, CNN_classes_cupy.py:622-626) goes to the
    kernels as dense float32 rows."""
    import numpy as np
    from aether.layers import _targets
    y = np.array([2, 0, 1])
    kind, t = _targets(y)
    assert kind == "index" and t.dtype == np.int32 and list(t) == [2, 0, 1]
    kind, t = _targets(np.eye(3)[y])
    assert kind == "index" and list(t) == [2, 0, 1]
    soft = np.eye(3)[y] * 0.9 + 0.1 / 3
    kind, t = _targets(soft)
    assert kind == "dense" and t.dtype == np.float32 and t.shape == (3, 3) and np.allclose(t, soft)
    kind, t = _targets(np.array([[1.0, 1.0, 0.0]]))
    assert kind == "dense"


def test_accuracy_classes_follow_the_reference():
    """Accuracy_Regression (CNN_model_cupy.py:367-378): correct within std(y)/250, a precision kept until
    `reinit`; Accuracy_Categorical (:380-387): one-hot targets are reduced to indices.  Host-only classes."""
    import numpy as np
    import aether
    assert set(aether.__all__) >= {"Accuracy", "Accuracy_Regression", "Accuracy_Categorical", "Layer_Input", "Model"}
    y = np.array([[0.0], [250.0], [500.0]])
    acc = aether.Accuracy_Regression()
    acc.init(y)
    assert acc.precision == np.std(y) / 250
    acc.new_pass()
    hits = acc.calculate(y + np.array([[0.5], [-0.9], [0.1]]), y)      # precision = 0.8165
    assert hits == 2 / 3
    acc.calculate(y, y)
    assert acc.calculate_accumulated() == 5 / 6
    acc.init(y * 2)
    assert acc.precision == np.std(y) / 250                 # kept
    acc.init(y * 2, reinit=True)
    assert acc.precision == np.std(y * 2) / 250
    cat = aether.Accuracy_Categorical()
    cat.new_pass()
    assert cat.calculate(np.array([2, 0, 1]), np.eye(3)[[2, 1, 1]]) == 2 / 3


def test_debug_switches_are_known_by_name(lib):
    """aeth_debug_set may be called before aeth_init: known names are accepted, -1 and NULL reset,
    an unknown name is refused with a message that names it."""
    for name in (b"gather_bm", b"gather_kc", b"gather_nloop", b"gather_halo", b"gather_split", b"gather_sa",
                 b"gather_direct_b", b"gather_clip", b"gather_merge", b"gather_pairs", b"gather_runs", b"narrow", b"gather_bkn", b"gather_wide", b"gather_res", b"dense_res", b"direct",
                 b"wgrad_halo", b"wgrad_wide", b"wgrad_cw", b"wgrad_br", b"wgrad_rounds", b"wgrad_swap", b"gather_border", b"pair_bwd"):
        assert lib.aeth_debug_set(name, 1) == 0, name
        assert lib.aeth_debug_set(name, -1) == 0, name
    assert lib.aeth_debug_set(None, 0) == 0
    assert lib.aeth_debug_set(b"no_such_switch", 1) == -1
    assert b"no_such_switch" in lib.aeth_last_error()
    # every name the header lists is one the library knows
    text = open(HEADER).read()
    doc = text[text.index("Names:"):text.index("May be called before aeth_init")]
    for name in doc.replace("Names:", "").replace("*", " ").replace(".", " ").replace(",", " ").split():
        assert lib.aeth_debug_set(name.encode(), -1) == 0, name
