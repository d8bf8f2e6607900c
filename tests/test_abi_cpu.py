"""CPU-only checks of the C-ABI boundary: the shared library loads, exports every symbol
include/haste_hip.h declares, and rejects bad arguments before touching the GPU."""
import ctypes
import os
import re

import pytest

from haste_amd import lib as hlib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(hlib.LIB_PATH):
        from haste_amd import build
        build.build(force=True)
    return hlib.load()


def test_library_exports_every_declared_symbol(lib):
    names = hlib.declared_symbols()
    assert len(names) >= 25
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_version_and_error_strings(lib):
    assert lib.haste_hip_version() >= 100
    for code in range(0, 5):
        assert lib.haste_hip_error_string(code)
    assert b"unknown" in lib.haste_hip_error_string(99)


def _call(lib, name, *args):
    fn = getattr(lib, name)
    fn.restype = ctypes.c_int
    conv = []
    for a in args:
        if a is None:
            conv.append(ctypes.c_void_p(0))
        elif isinstance(a, float):
            conv.append(ctypes.c_float(a))
        else:
            conv.append(ctypes.c_int(a))
    return fn(*conv)


def test_null_pointers_and_bad_dimensions_are_rejected_on_the_host(lib):
    INVALID = 1
    # gemm: null operands, non-positive sizes
    assert _call(lib, "haste_hip_gemm_f32", 0, 4, 4, 4, None, 4, None, 4, None, 4, 0, None) == INVALID
    assert _call(lib, "haste_hip_gemm_f32", 0, 0, 4, 4, None, 4, None, 4, None, 4, 0, None) == INVALID
    # every cell: zero steps / null tensors
    assert _call(lib, "haste_hip_lstm_forward_f32", 1, 0, 1, 1, 1, *([None] * 8), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_lstm_forward_f32", 1, 3, 2, 2, 2, *([None] * 8), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_lstm_backward_f32", 3, 2, 2, 2, *([None] * 16), None) == INVALID
    assert _call(lib, "haste_hip_gru_forward_f32", 1, 3, 2, 2, 2, *([None] * 9), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_gru_backward_f32", 3, 2, 2, 2, *([None] * 17), None) == INVALID
    assert _call(lib, "haste_hip_transpose3_f32", *([4, 4, None, None] * 3), None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_forward_f32", 4, 8, *([None] * 5), None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_backward_f32", 4, 8, *([None] * 7), None) == INVALID
    assert _call(lib, "haste_hip_indrnn_forward_f32", 1, 3, 2, 2, 2, *([None] * 6), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_indrnn_backward_f32", 3, 2, 2, 2, *([None] * 13), None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_lstm_forward_f32", 1, 3, 2, 2, 2, *([None] * 18), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_gru_forward_f32", 1, 3, 2, 2, 2, *([None] * 15), 0.0, None, None) == INVALID


def test_double_and_half_entry_points_reject_bad_arguments_too(lib):
    INVALID = 1
    for sfx in ("_f64", "_f16"):
        assert _call(lib, "haste_hip_gemm" + sfx, 0, 4, 4, 4, None, 4, None, 4, None, 4, 0, None) == INVALID
        assert _call(lib, "haste_hip_transpose" + sfx, 4, 4, None, None, None) == INVALID
        assert _call(lib, "haste_hip_gru_forward" + sfx, 1, 0, 1, 1, 1, *([None] * 9), 0.0, None, None) == INVALID
        assert _call(lib, "haste_hip_gru_forward" + sfx, 1, 3, 2, 2, 2, *([None] * 9), 0.0, None, None) == INVALID
        assert _call(lib, "haste_hip_gru_backward" + sfx, 3, 2, 2, 2, *([None] * 17), None) == INVALID
    assert _call(lib, "haste_hip_lstm_forward_f64", 1, 3, 2, 2, 2, *([None] * 8), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_lstm_backward_f64", 3, 2, 2, 2, *([None] * 16), None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_forward_f64", 4, 8, *([None] * 5), None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_backward_f64", 4, 8, *([None] * 7), None) == INVALID
    assert _call(lib, "haste_hip_indrnn_forward_f64", 1, 3, 2, 2, 2, *([None] * 6), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_lstm_forward_f64", 1, 3, 2, 2, 2, *([None] * 18), 0.0, None, None) == INVALID
    assert _call(lib, "haste_hip_layer_norm_gru_forward_f64", 1, 3, 2, 2, 2, *([None] * 15), 0.0, None, None) == INVALID
    # as in the reference, half exists for the GRU only
    assert not hasattr(lib, "haste_hip_lstm_forward_f16")


def test_cpp_headers_declare_the_reference_class_surface():
    """include/haste/*.h keeps the reference's namespaces and class names."""
    for ns in ("lstm", "gru", "indrnn", "layer_norm", "layer_norm_lstm", "layer_norm_gru",
               "layer_norm_indrnn"):
        text = open(os.path.join(ROOT, "include", "haste", ns + ".h")).read()
        assert re.search(r"namespace %s \{" % ns, text)
        assert "class ForwardPass" in text and "class BackwardPass" in text
        assert "void Run(" in text
