"""The C-ABI library loads and exports every symbol the public headers declare.
No compute call is made here, so this runs without a GPU."""
import ctypes
import os
import re

from darknet_amd import lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # comments
    text = re.sub(r"(?m)^\s*#.*$", "", text)                    # preprocessor
    text = re.sub(r"\{[^{}]*\}", "{}", text)                    # struct / enum bodies
    text = re.sub(r"\{[^{}]*\}", "{}", text)
    names = set()
    for stmt in text.split(";"):
        m = re.search(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^()]*(\([^()]*\)[^()]*)*\)\s*$", stmt.strip())
        if m and "typedef" not in stmt and "(*" not in stmt.split("(")[0]:
            names.add(m.group(1))
    return names


def test_library_exports_every_declared_entry_point():
    L = ctypes.CDLL(lib.LIB_PATH)
    hip = declared("darknet_hip.h")
    amd = declared("darknet_amd.h")
    assert {"hip_make_array", "cuda_make_array", "forward_convolutional_gpu", "fill_gpu", "im2col_gpu"} <= hip
    assert {"parse_network_cfg", "network_predict", "make_convolutional_layer",
            "forward_convolutional_layer_gpu"} <= amd
    missing = [n for n in sorted(hip | amd) if not hasattr(L, n)]
    assert not missing, missing
    ctypes.c_int.in_dll(L, "gpu_index")


def test_python_bindings_cover_the_headers():
    bound = set(lib.SIGNATURES) | set(lib.STRUCT_BY_VALUE)
    missing = sorted((declared("darknet_hip.h") | declared("darknet_amd.h")) - bound)
    assert not missing, missing
    lib.load()


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    monkeypatch.setattr(lib, "LIB_PATH", str(tmp_path / "nope.so"))
    monkeypatch.setattr(lib, "_lib", None)
    try:
        lib.load()
    except RuntimeError as e:
        assert "no fallback" in str(e)
    else:
        raise AssertionError("load() must raise when the shared object is absent")
