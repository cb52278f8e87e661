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


def _collects(handle, shape, strides):
    from rmlk_amd._lib import Dims
    handle.rmlk_hip_batch_collects.restype = ctypes.c_int32
    handle.rmlk_hip_batch_collects.argtypes = [ctypes.POINTER(Dims), ctypes.c_int32, ctypes.POINTER(Dims)]
    arr = (Dims * len(strides))(*[Dims.of(s) for s in strides])
    return handle.rmlk_hip_batch_collects(Dims.of(shape), len(strides) - 1, arr)


def test_collected_launches_refuse_offsets_beyond_32_bits(handle):
    """A record of the collected launch keeps 32-bit element strides and the kernel adds offsets up
    in 32 bits: a tiny tensor whose operand strides reach 2^31 elements must be launched as usual
    (host arithmetic only, nothing runs)."""
    dense = [32, 1]
    assert _collects(handle, [32, 32], [dense, dense, dense]) == 1
    assert _collects(handle, [32, 32], [dense, [0, 1], dense]) == 1            # broadcast operand
    assert _collects(handle, [1024, 1024], [[1024, 1]] * 3) == 0               # too many elements
    # 1024 elements, each stride below 2^30, but the last element lies 31 * 2^27 + 31 * 2^21 > 2^31 away
    far = [1 << 27, 1 << 21]
    assert (32 - 1) * far[0] + 31 * far[1] >= 1 << 31
    assert _collects(handle, [32, 32], [far, dense, dense]) == 0
    assert _collects(handle, [32, 32], [dense, dense, far]) == 0               # the output too
    near = [1 << 25, 1 << 20]                                                  # reach just under 2^30
    assert _collects(handle, [32, 32], [near, dense, dense]) == 1
    assert _collects(handle, [2, 2], [[1 << 31, 1], [2, 1], [2, 1]]) == 0      # one stride beyond 2^30
    assert _collects(handle, [2, 2], [[-(1 << 30), 1], [2, 1], [2, 1]]) == 1   # negative strides count by size
