"""`@kernel` decorator: trace a Python function into a DVM kernel once, call it with numpy arrays or with
torch tensors that live on the GPU (those are used in place, see JitKernel._call_on_tensors).

Same contract as the reference's python/dvm/jit.py:20-78: the decorated
function receives the kernel object and one placeholder index per argument;
`k.load(idx, dtype)`, `k.scalar(idx)` and `k.int_array(idx)` declare what each
argument is; calling the result binds the arguments, (re)generates code for a
dynamic kernel, runs it and returns the stored outputs as numpy arrays.
"""
import os

from ._core import PyKernel, DataType


class JitKernel(PyKernel):
    def __init__(self, ker_type, dynamic, run_type="dev"):
        if dynamic:
            ker_type += ",dyn" if ":" in ker_type else ":dyn"
        dev_conf = os.getenv("DEVICE_ID")
        dev_id = int(dev_conf) if dev_conf else 0
        PyKernel.__init__(self, ker_type, run_type, dev_id)
        self.inputs = None
        self.outputs = None
        self.dynamic = dynamic

    def build(self, func):
        arg_cnt = func.__code__.co_argcount - 1
        self.inputs = [None] * arg_cnt
        self.outputs = func(self, *range(arg_cnt))
        if not self.dynamic:
            self.codegen(None)

    def load(self, index, dtype, shape=()):
        op = PyKernel.load(self, list(shape), dtype)
        self.inputs[index] = op
        return op

    def scalar(self, index, dtype=DataType.float32):
        ref = PyKernel.scalar(self, dtype)
        self.inputs[index] = ref
        return ref

    def int_array(self, index):
        ref = PyKernel.int_array(self)
        self.inputs[index] = ref
        return ref

    def __call__(self, *args):
        if any(_is_device_tensor(a) for a in args):
            return self._call_on_tensors(args)
        for inp, arg in zip(self.inputs, args):
            PyKernel.input(self, inp, arg)
        if self.dynamic:
            self.codegen(None)
        self.run()
        if isinstance(self.outputs, (list, tuple)):
            return [self.output(x) for x in self.outputs]
        return self.output(self.outputs)


    def _call_on_tensors(self, args):
        """torch tensors on the GPU as arguments: nothing is copied. Inputs are read where they are, outputs are
        new torch tensors, and the launches go to torch's current stream without waiting for them (the caller
        orders later work like after any torch operator). Scalars and shape lists are passed as usual."""
        import torch
        dev = None
        keep = []
        for inp, arg in zip(self.inputs, args):
            if not _is_device_tensor(arg):
                if isinstance(arg, torch.Tensor):
                    raise TypeError("tensor arguments have to live on the GPU, all of them")
                PyKernel.input(self, inp, arg)
                continue
            want = _TORCH_DTYPES()[int(inp.dtype())]
            if arg.dtype != want:
                raise TypeError("argument is %s, the kernel's load is %s" % (arg.dtype, want))
            t = arg.contiguous()
            keep.append(t)
            dev = t.device
            self.bind_device(inp, t.data_ptr(), tuple(t.shape))
        self.normalize()
        single = not isinstance(self.outputs, (list, tuple))
        outs = []
        for st in ([self.outputs] if single else self.outputs):
            o = torch.empty(tuple(st.shape()), dtype=_TORCH_DTYPES()[int(st.dtype())], device=dev)
            self.bind_device(st, o.data_ptr())
            outs.append(o)
        self.codegen(None)  # addresses are part of the programs, so also for a kernel of fixed shapes
        self.run(stream=torch.cuda.current_stream(dev).cuda_stream, sync=False)
        self._alive = keep + outs  # until the next call: the launches may still be running
        return outs[0] if single else outs


def _is_device_tensor(a):
    return hasattr(a, "data_ptr") and getattr(a, "is_cuda", False)


def _TORCH_DTYPES():
    import torch
    return {int(DataType.bool): torch.bool, int(DataType.float16): torch.float16, int(DataType.bfloat16): torch.bfloat16,
            int(DataType.float32): torch.float32, int(DataType.int32): torch.int32}


def kernel(ktype="split", dynamic=True, run_type="dev"):
    if callable(ktype):
        kobj = JitKernel("split", True)
        kobj.build(ktype)
        return kobj

    def decorate(func):
        kobj = JitKernel(ktype, dynamic, run_type)
        kobj.build(func)
        return kobj

    return decorate
