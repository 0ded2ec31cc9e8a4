"""The C-ABI library loads on a CPU-only host and exports every symbol include/sofie_hip.h declares
(no compute is called here)."""
import ctypes
import os
import re

from sofie_amd import lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    with open(os.path.join(ROOT, "include", "sofie_hip.h")) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    return sorted(set(re.findall(r"\b(sofie_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_expects():
    assert set(declared_symbols()) == set(lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(lib.LIB_PATH), "libsofie_hip.so has not been built"
    dll = ctypes.CDLL(lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(dll, name), name
    assert lib.load().sofie_hip_version() >= 1


def test_null_context_is_rejected_without_touching_a_gpu():
    l = lib.load()
    assert l.sofie_hip_sync(None) == lib.EINVAL
    assert l.sofie_hip_relu_f32(None, None, None, 4) == lib.EINVAL
    assert l.sofie_hip_last_error(None) == b"null context"
