"""MI355X (gfx950) kernels for llmpalooza's quantized linear-layer path.

The product is the C-ABI shared library built from csrc/ (declared in
include/llmp_hip.h). This package is its Python host side: a ctypes binding
(`_lib`), operator wrappers over device memory held in torch tensors (`ops`),
and seeded synthetic inputs of the benchmark shapes (`synth`).
"""
from . import _lib  # noqa: F401

__all__ = ["_lib", "ops", "synth"]
