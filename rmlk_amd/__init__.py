"""rmlk_amd: gfx950 (MI355X) kernel backend for the rmlk ONNX runtime's operator path.

`rmlk_amd.kernels` mirrors the reference's kernel crate (`rmlk_cuda::kernels::*`) over the C ABI of
`librmlk_hip.so`; `rmlk_amd.runtime` mirrors its operator dispatch and graph execution. Nothing in
this package computes on the CPU: without the built HIP library every call raises.
"""
from ._lib import LibraryNotBuilt, RmlkError, lib, library_path  # noqa: F401

__version__ = "0.1.0"
