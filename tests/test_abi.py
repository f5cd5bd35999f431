"""The C-ABI library loads without a GPU and exports every symbol the header declares.
No compute calls here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tilefusion_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tf_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(tf):
    lib = C.CDLL(tf.lib_path())
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in tilefusion_hip.h but not exported"


def test_binding_covers_the_header(tf):
    from importlib import import_module
    binding = import_module("tile-fusion_amd.binding")
    assert sorted(binding.SIGNATURES) == declared_symbols()


def test_version_and_error_channel(tf):
    lib = tf.lib()
    assert lib.tf_version().decode() == "0.1"
    # a null output pointer is rejected before any device work
    assert lib.tf_inspect(4, 4, None, None, None, None) == -1
    assert b"tf_inspect" in lib.tf_last_error_string()
    # the issue probe checks its roles and rounds before it touches the device
    ms = C.c_float(-1.0)
    assert lib.tf_calibrate_issue(4, 0, 10, C.byref(ms)) == -1 and lib.tf_calibrate_issue(1, 2, 0, C.byref(ms)) == -1
    assert lib.tf_calibrate_issue(1, 2, 10, None) == -1 and ms.value == -1.0
    assert b"tf_calibrate_issue" in lib.tf_last_error_string()


def test_cpp_header_compiles(tmp_path):
    """include/tile-fusion.h is self-contained C++17 and names the README API."""
    import subprocess
    src = tmp_path / "t.cpp"
    src.write_text('#include "tile-fusion.h"\n'
                   "using namespace swiftware;\n"
                   "void f(def::CSRMatrix A, def::Matrix B, def::Matrix C, def::Matrix D) {\n"
                   "  def::FusedSchedule s = fusion::inspector(A, 8);\n"
                   "  fusion::geMMSpMMExecutor(A, B, C, D, s, 8);\n"
                   "  fusion::spMMSpMMExecutor(A, A, C, D, s, 8);\n"
                   "}\n")
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(src)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
