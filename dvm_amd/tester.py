"""Test harness with the interface of the reference's python/dvm/tester.py:70-431.

A test builds a graph with `load` (numpy array in, or a shape for dynamic
kernels), computes its expectation with NumPy inline, registers it with
`store_expect` and calls `run_check`, which compares with
np.allclose(rtol=eps, atol=eps, equal_nan=True); default eps 1e-5 for fp32,
1e-3 for fp16, 0 otherwise.
"""
import inspect
import os
import sys

import numpy as np

from ._core import DataType, PyKernel, Device

_DTYPE_NAME_MAP = {
    "bool": DataType.bool,
    "float16": DataType.float16,
    "bfloat16": DataType.bfloat16,
    "float32": DataType.float32,
    "int32": DataType.int32,
    "int64": DataType.int64,
}


def _normalize_dtype(dtype):
    if isinstance(dtype, DataType):
        return dtype
    if isinstance(dtype, str):
        if dtype not in _DTYPE_NAME_MAP:
            raise ValueError("Unsupported dtype string: %s" % dtype)
        return _DTYPE_NAME_MAP[dtype]
    if dtype is not None and not isinstance(dtype, int):
        return _normalize_dtype(np.dtype(dtype).name)
    return dtype


class PerformanceResult:
    def __init__(self, results):
        self.min, self.max, self.mean = results

    def __repr__(self):
        return "min_max_avg(us): %.2f %.2f %.2f" % (self.min, self.max, self.mean)


class Tester(PyKernel):
    __test__ = False

    def __init__(self, ker_type="", use_pass_opt=False, run_mode="dev"):
        dev_conf = os.getenv("DEVICE_ID")
        PyKernel.__init__(self, ker_type, run_mode, int(dev_conf) if dev_conf else 0)
        self.is_dyn = "dyn" in ker_type
        self.is_codegen = False
        self.expects = []  # [op, expect, eps]
        self.passes = None if use_pass_opt else []

    @staticmethod
    def fast_random_normal(loc, scale, shape):
        row = np.random.normal(loc, scale, (shape[-1],)).astype(np.float32)
        return np.broadcast_to(row, shape).copy()

    @staticmethod
    def bf16_random_normal(loc, scale, shape):
        x = np.random.normal(loc, scale, shape).astype(np.float32)
        return (x.view(np.uint32) & 0xFFFF0000).view(np.float32)

    def _prepare_array_input(self, array, dtype):
        dtype_id = _normalize_dtype(str(array.dtype)) if dtype is None else _normalize_dtype(dtype)
        if dtype_id == DataType.bfloat16:
            array = PyKernel.convert_to_bf16(array)
        return array, dtype_id, list(array.shape)

    def load(self, shape_arr, dtype=None):
        if not isinstance(shape_arr, np.ndarray):
            return PyKernel.load(self, shape_arr, _normalize_dtype(dtype))  # dynamic shape
        shape_arr, dtype_id, shape = self._prepare_array_input(shape_arr, dtype)
        op = PyKernel.load(self, shape, dtype_id)
        self.input(op, shape_arr)
        return op

    # views: the array bound to the load is the whole buffer, the load reads part of it
    def view_load(self, shape, stride, arr_dtype, offset=0, real_dtype=None):
        if not isinstance(arr_dtype, np.ndarray):
            return PyKernel.view_load(self, shape, stride, _normalize_dtype(arr_dtype))  # dynamic shape
        arr, dtype_id, _ = self._prepare_array_input(arr_dtype, real_dtype)
        op = PyKernel.view_load(self, shape, stride, dtype_id)
        self.input(op, arr, offset)
        return op

    def slice_load(self, shape_arr, start, size, dtype=None):
        if not isinstance(shape_arr, np.ndarray):
            return PyKernel.slice_load(self, shape_arr, start, size, _normalize_dtype(dtype))
        arr, dtype_id, shape = self._prepare_array_input(shape_arr, dtype)
        op = PyKernel.slice_load(self, shape, start, size, dtype_id)
        self.input(op, arr)
        return op

    def stridedslice_load(self, shape_arr, start, end, step, dtype=None):
        if not isinstance(shape_arr, np.ndarray):
            return PyKernel.stridedslice_load(self, shape_arr, start, end, step, _normalize_dtype(dtype))
        arr, dtype_id, shape = self._prepare_array_input(shape_arr, dtype)
        op = PyKernel.stridedslice_load(self, shape, start, end, step, dtype_id)
        self.input(op, arr)
        return op

    def view_store_expect(self, x, stride, e, eps=None):
        """Stores x through `stride` into a buffer shaped like e (zeros where nothing is written) and expects e."""
        e = np.asarray(e)
        op = PyKernel.view_store(self, x, stride, e.size)
        self._view_shape = getattr(self, "_view_shape", {})
        self._view_shape[op._h] = tuple(e.shape)
        self.expects.append([op, e, eps])
        return op

    def output(self, store, shape=None):
        if shape is None:
            shape = getattr(self, "_view_shape", {}).get(store._h)
        return PyKernel.output(self, store, shape)

    def cast(self, x, dtype):
        return PyKernel.cast(self, x, _normalize_dtype(dtype))

    def full(self, scalar, shape, dtype=None):
        return PyKernel.full(self, scalar, shape, _normalize_dtype(dtype))

    def store_expect(self, x, e, eps=None):
        op = PyKernel.store(self, x)
        self.expects.append([op, e, eps])
        return op

    def dump_verbose(self):
        print("******* graph *******")
        print(self.dump())
        print("********* bytecode *********")
        print(self.das())

    def codegen(self, verbose=False):
        if self.is_codegen:
            return
        PyKernel.codegen(self, self.passes)
        if verbose:
            self.dump_verbose()
        if not self.is_dyn:
            self.is_codegen = True

    def run(self, verbose=False):
        self.codegen()
        PyKernel.run(self)
        if verbose:
            self.dump_verbose()

    def bare_run(self):
        PyKernel.run(self)

    def check(self, store, expect, eps=None, verbose=False):
        out = self.output(store)
        if store.dtype() == DataType.bfloat16:
            out = PyKernel.convert_from_bf16(out)
        if inspect.isfunction(expect):
            ok = bool(expect(out))
        else:
            if eps is None:
                eps = 1e-5 if out.dtype == np.float32 else (1e-3 if out.dtype == np.float16 else 0)
            ok = bool(np.allclose(out, expect, rtol=eps, atol=eps, equal_nan=True))
        if not ok and verbose:
            print("********** OUTPUT **********", file=sys.stderr)
            print(out, file=sys.stderr)
            print("********** EXPECT **********", file=sys.stderr)
            print(expect, file=sys.stderr)
        return ok

    def run_check(self, verbose=False):
        self.run(verbose)
        for op, expect, eps in self.expects:
            if not self.check(op, expect, eps, verbose):
                return False
        return True

    def run_perf(self):
        self.codegen()
        return PerformanceResult(self.perf())

    def set_passes(self, *pass_names):
        self.passes = list(pass_names)

    def reset(self):
        PyKernel.reset(self)
        self.is_codegen = False
        self.expects = []
