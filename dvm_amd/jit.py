"""`@kernel` decorator: trace a Python function into a DVM kernel once, call it with numpy arrays.

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
        for inp, arg in zip(self.inputs, args):
            PyKernel.input(self, inp, arg)
        if self.dynamic:
            self.codegen(None)
        self.run()
        if isinstance(self.outputs, (list, tuple)):
            return [self.output(x) for x in self.outputs]
        return self.output(self.outputs)


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
