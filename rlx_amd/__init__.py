"""rlx_amd: MI355X (gfx950) backend for RLX's GGUF dequant-matmul and FakeQuantize path.

The product is librlx_mi355x.so (C ABI in include/rlx_mi355x.h, HIP kernels in rlx_amd/csrc/kernels). This package is
the thin host-side mirror of the reference's Session / Graph surface used by tests and bench.py."""
from . import _lib, gguf, ops
from ._lib import RlxError, build
from .ir import DType, Graph, Op, OpKind, QuantScheme, RoundMode, ScaleMode, Shape, SteKind
from .runtime import CompiledGraph, Device, Session, is_available, launch_sequence, supported_ops

__all__ = ["_lib", "gguf", "ops", "RlxError", "build", "DType", "Graph", "Op", "OpKind", "QuantScheme", "RoundMode", "ScaleMode",
           "Shape", "SteKind", "CompiledGraph", "Device", "Session", "is_available", "launch_sequence", "supported_ops"]
