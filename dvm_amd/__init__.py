"""dvm_amd: MI355X (gfx950) backend of the DVM fused-operator JIT.

Python surface of the reference package `dvm` (python/dvm/__init__.py:17-42):
the `kernel` decorator, the dtype aliases and the builder/runner classes.
Typical use: `import dvm_amd as dvm`.
"""
from ._core import DataType, Device, Kernel, PyKernel, NDObject, IntArrayRef, ScalarRef
from .jit import kernel

bool_ = DataType.bool
float16 = DataType.float16
bfloat16 = DataType.bfloat16
float32 = DataType.float32
int32 = DataType.int32
int64 = DataType.int64

__all__ = ["DataType", "Device", "Kernel", "PyKernel", "NDObject", "IntArrayRef", "ScalarRef", "kernel",
           "bool_", "float16", "bfloat16", "float32", "int32", "int64"]
