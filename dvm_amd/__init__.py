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



def lazy_fusion(ktype="eager"):
    """Eager fusion without graphs for PyTorch tensors on the GPU (dvm_amd/lazy.py); imports torch on first use."""
    from .lazy import lazy_fusion as _lazy_fusion
    return _lazy_fusion(ktype)


__all__ = ["lazy_fusion", "DataType", "Device", "Kernel", "PyKernel", "NDObject", "IntArrayRef", "ScalarRef", "kernel",
           "bool_", "float16", "bfloat16", "float32", "int32", "int64"]
