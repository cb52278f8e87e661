"""The shared library loads without a GPU and exports every entry point the headers declare; the
ctypes binding table covers the same set. No compute call is made here."""
import ctypes
import os
import re

import pytest

import rmlk_amd
from rmlk_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DECL = re.compile(r"^\s*(?:RMLK_API\s+)?(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(rmlk_[a-z0-9_]+)\s*\(", re.M)


def declared_symbols():
    names = set()
    for header in ("rmlk_hip.h", "rmlk_runtime.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for m in DECL.finditer(text):
            name = m.group(1)
            if not name.endswith("_t"):
                names.add(name)
    return names


@pytest.fixture(scope="module")
def handle():
    path = rmlk_amd.library_path()
    if not os.path.exists(path):
        pytest.fail(f"{path} is not built: run `make -C rmlk_amd/csrc`")
    return ctypes.CDLL(path)


def test_headers_declare_something():
    names = declared_symbols()
    assert "rmlk_hip_matmul" in names and "rmlk_session_run" in names
    assert len(names) >= 50


def test_library_exports_every_declared_symbol(handle):
    missing = sorted(n for n in declared_symbols() if not hasattr(handle, n))
    assert not missing, f"declared in include/ but not exported: {missing}"


def test_binding_table_matches_headers():
    declared = declared_symbols()
    bound = set(_lib.SIGNATURES)
    assert not (declared - bound), f"declared but not bound in _lib.SIGNATURES: {sorted(declared - bound)}"
    assert not (bound - declared), f"bound but not declared in include/: {sorted(bound - declared)}"


def test_version_and_status_strings_without_gpu(handle):
    handle.rmlk_hip_version.restype = ctypes.c_char_p
    assert handle.rmlk_hip_version().decode().count(".") == 2
    handle.rmlk_hip_status_string.restype = ctypes.c_char_p
    handle.rmlk_hip_status_string.argtypes = [ctypes.c_int32]
    assert "dtype" in handle.rmlk_hip_status_string(-2).decode().lower() or \
        handle.rmlk_hip_status_string(-2).decode()
