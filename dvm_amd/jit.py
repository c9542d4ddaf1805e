"""`@kernel`: trace a Python function into a DVM kernel once, then call it like a function.

Public contract of the reference's python/dvm/jit.py:20-78: the decorated function receives the kernel object
and one placeholder per argument (its position); `k.load(idx, dtype)`, `k.scalar(idx)` and `k.int_array(idx)`
say what the argument at that position is; a call binds the arguments, generates code again when the kernel
is dynamic, runs, and returns the stored outputs (one array, or a list when the function returned several).

Arguments may be numpy arrays (copied to the device and back) or torch tensors that live on the GPU (read and
written in place, launched on torch's current stream; see `_DeviceCall`). With torch tensors a call also takes
`out=` (a tensor, or a sequence of them: the outputs are written there instead of into new tensors, the call form
of the reference's docs/pytorch.md:238-239), reads tensors that are not contiguous through their strides, and takes
its workspace from torch's caching allocator.
"""
import inspect
import os

from ._core import PyKernel, DataType


class _Slot:
    """What one positional argument of the traced function turned out to be."""

    __slots__ = ("role", "handle")

    def __init__(self, role, handle):
        self.role, self.handle = role, handle  # role: "tensor", "scalar" or "ints"


class JitKernel(PyKernel):
    def __init__(self, ker_type, dynamic, run_type="dev"):
        spec = ker_type
        if dynamic:
            spec += (",dyn" if ":" in ker_type else ":dyn")
        PyKernel.__init__(self, spec, run_type, int(os.getenv("DEVICE_ID") or 0))
        self.dynamic = bool(dynamic)
        self._slots = []      # one _Slot per argument, filled while tracing
        self._results = None  # what the traced function returned: a store or a sequence of stores

    # ---- tracing ----
    def build(self, func):
        positional = [p for p in inspect.signature(func).parameters.values()
                      if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
        self._slots = [None] * (len(positional) - 1)  # the first parameter is the kernel itself
        self._results = func(self, *range(len(self._slots)))
        missing = [i for i, s in enumerate(self._slots) if s is None]
        if missing:
            raise TypeError("%s never declared what argument(s) %s are (k.load / k.scalar / k.int_array)"
                            % (getattr(func, "__name__", "kernel"), missing))
        if not self.dynamic:
            self.codegen()

    def _declare(self, index, role, handle):
        if not 0 <= index < len(self._slots):
            raise IndexError("placeholder %d is not an argument of the traced function" % index)
        self._slots[index] = _Slot(role, handle)
        return handle

    def load(self, index, dtype, shape=()):
        return self._declare(index, "tensor", PyKernel.load(self, list(shape), dtype))

    def scalar(self, index, dtype=DataType.float32):
        return self._declare(index, "scalar", PyKernel.scalar(self, dtype))

    def int_array(self, index):
        return self._declare(index, "ints", PyKernel.int_array(self))

    # ---- calling ----
    def _stores(self):
        many = isinstance(self._results, (list, tuple))
        return (list(self._results) if many else [self._results]), many

    def __call__(self, *args, out=None):
        if len(args) != len(self._slots):
            raise TypeError("kernel takes %d arguments, %d given" % (len(self._slots), len(args)))
        if any(_on_gpu(a) for a in args):
            return _DeviceCall(self, args, out).run()
        if out is not None:
            raise TypeError("out= takes torch tensors on the GPU, beside arguments that are such tensors")
        self.release_device_bindings()  # a call on torch tensors before this one left their addresses behind
        self.set_workspace_allocator(None)
        for slot, value in zip(self._slots, args):
            self.input(slot.handle, value)
        if self.dynamic:
            self.codegen()
        self.run()
        stores, many = self._stores()
        arrays = [self.output(s) for s in stores]
        return arrays if many else arrays[0]


class _DeviceCall:
    """One call of a JitKernel on torch tensors that live on the GPU. Nothing is copied: loads read the tensors'
    memory (through their strides when they are not contiguous; only a view the kernel cannot walk in place is made
    contiguous first), every store gets a fresh torch tensor of the inferred shape or the caller's `out=` tensor, the
    workspace comes from torch's allocator, and the launches go to torch's current stream without a
    synchronisation, like any torch operator. Scalars and shape lists are bound as usual."""

    def __init__(self, kern, args, out=None):
        import torch
        self.torch, self.kern, self.args, self.out = torch, kern, args, out
        self.types = {int(DataType.bool): torch.bool, int(DataType.float16): torch.float16,
                      int(DataType.bfloat16): torch.bfloat16, int(DataType.float32): torch.float32,
                      int(DataType.int32): torch.int32, int(DataType.int64): torch.int64}

    def _bind_inputs(self, in_place):
        """Binds the arguments; `in_place`: tensors that are not contiguous are read through their strides,
        otherwise a contiguous copy is bound. Returns (tensors to keep alive, device)."""
        torch, k = self.torch, self.kern
        held, device = [], None
        for slot, value in zip(k._slots, self.args):
            if slot.role != "tensor" or not _on_gpu(value):
                if isinstance(value, torch.Tensor):
                    raise TypeError("tensor arguments have to live on the GPU, all of them")
                k.input(slot.handle, value)
                continue
            want = self.types[int(slot.handle.dtype())]
            if value.dtype != want:
                raise TypeError("argument is %s, the kernel's load is %s" % (value.dtype, want))
            device = value.device
            walkable = value.dim() > 0 and all(s >= 0 for s in value.stride()) and value.numel() > 0
            if value.is_contiguous() or not (in_place and walkable):
                value = value.contiguous()
                k.bind_device(slot.handle, value.data_ptr(), tuple(value.shape))
            else:
                k.bind_device(slot.handle, value.data_ptr(), tuple(value.shape), strides=tuple(value.stride()))
            held.append(value)
        return held, device

    def _bind_outputs(self, device):
        torch, k = self.torch, self.kern
        stores, many = k._stores()
        given = None
        if self.out is not None:
            given = list(self.out) if isinstance(self.out, (list, tuple)) else [self.out]
            if len(given) != len(stores):
                raise TypeError("the kernel has %d outputs, out= holds %d" % (len(stores), len(given)))
        outs = []
        for i, st in enumerate(stores):
            shape, dtype = tuple(st.shape()), self.types[int(st.dtype())]
            if given is None:
                o = torch.empty(shape, dtype=dtype, device=device)
            else:
                o = given[i]
                if not _on_gpu(o) or o.dtype != dtype or tuple(o.shape) != shape or not o.is_contiguous():
                    raise TypeError("out[%d] has to be a contiguous %s tensor of shape %s on the GPU" % (i, dtype, list(shape)))
            k.bind_device(st, o.data_ptr())
            outs.append(o)
        return outs, many

    def run(self):
        torch, k = self.torch, self.kern
        for in_place in (True, False):
            held, device = self._bind_inputs(in_place)
            k.normalize()  # output shapes are known from here on
            outs, many = self._bind_outputs(device)
            # the workspace of the launches belongs to torch's caching allocator, like any temporary of an operator
            scratch = []

            def workspace(nbytes, scratch=scratch, device=device):
                scratch.append(torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device))
                return scratch[-1].data_ptr()

            k.set_workspace_allocator(workspace)
            try:
                k.codegen()  # addresses are part of the programs, so also for a kernel of fixed shapes
                break
            except RuntimeError as e:
                # a view the kernel cannot walk in place (a reshape of it, an operand without a contiguous axis):
                # once more on contiguous copies
                if not in_place or not any(s in str(e) for s in ("not supported", "needs a Copy")):
                    raise
        k.run(stream=torch.cuda.current_stream(device).cuda_stream, sync=False, on_given_stream=True)
        k._alive = held + outs + scratch  # until the next call: the launches may still be running
        return outs if many else outs[0]


def _on_gpu(value):
    return hasattr(value, "data_ptr") and bool(getattr(value, "is_cuda", False))


def kernel(ktype="split", dynamic=True, run_type="dev"):
    """`@kernel` or `@kernel(ktype=..., dynamic=..., run_type=...)`."""
    def trace(func, *conf):
        traced = JitKernel(*conf)
        traced.build(func)
        return traced

    if callable(ktype):  # used bare: the default split kernel with dynamic shapes
        return trace(ktype, "split", True)
    return lambda func: trace(func, ktype, dynamic, run_type)
