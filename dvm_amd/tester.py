"""Check harness over PyKernel with the public surface of the reference's python/dvm/tester.py:70-431
(`Tester.load / store_expect / run_check / run_perf / das / dump / set_passes`, `PerformanceResult`), so that a
test written against `dvm.tester` runs here unchanged.

How it is organised: every array that enters the graph goes through one `_HostArray` record (the numpy data as
the device wants it, the element type, the shape); every registered expectation is one `Expectation` record
that knows how to judge an output; the tolerance a dtype gets by default lives in `default_tolerance`, which
the parity tests share.
"""
import os
import sys
from collections import namedtuple

import numpy as np

from ._core import DataType, PyKernel

_BY_NAME = {"bool": DataType.bool, "float16": DataType.float16, "bfloat16": DataType.bfloat16,
            "float32": DataType.float32, "int32": DataType.int32, "int64": DataType.int64}


def as_datatype(spec):
    """DataType from a DataType, a name ("float16"), a numpy dtype or scalar type; None stays None."""
    if spec is None or isinstance(spec, DataType):
        return spec
    if isinstance(spec, int):
        return DataType(spec)
    name = spec if isinstance(spec, str) else np.dtype(spec).name
    try:
        return _BY_NAME[name]
    except KeyError:
        raise ValueError("Unsupported dtype string: %s" % name) from None


def default_tolerance(dtype):
    """rtol = atol used when a check names none: 1e-5 for fp32, 1e-3 for fp16, 1e-2 for bf16, exact otherwise
    (python/dvm/tester.py:322-330 for the first two; bf16 keeps 8 bits of mantissa)."""
    return {int(DataType.float32): 1e-5, int(DataType.float16): 1e-3, int(DataType.bfloat16): 1e-2}.get(int(as_datatype(dtype)), 0)


_HostArray = namedtuple("_HostArray", "data dtype shape")


def _host_array(array, dtype):
    """The bytes a load of element type `dtype` (default: the array's own) is fed with."""
    dt = as_datatype(array.dtype.name if dtype is None else dtype)
    data = PyKernel.convert_to_bf16(array) if dt == DataType.bfloat16 else array
    return _HostArray(data, dt, [int(d) for d in data.shape])


class Expectation:
    """What one stored output has to look like: a NumPy value compared with allclose, or a predicate."""

    __slots__ = ("store", "want", "eps", "buffer_shape")

    def __init__(self, store, want, eps=None, buffer_shape=None):
        self.store, self.want, self.eps, self.buffer_shape = store, want, eps, buffer_shape

    def holds(self, got):
        if callable(self.want) and not isinstance(self.want, np.ndarray):
            return bool(self.want(got))
        eps = self.eps
        if eps is None:
            # the reference judges by the dtype of the array it compares (bf16 outputs arrive widened to fp32)
            eps = 1e-5 if got.dtype == np.float32 else (1e-3 if got.dtype == np.float16 else 0)
        return bool(np.allclose(got, self.want, rtol=eps, atol=eps, equal_nan=True))


class PerformanceResult:
    """Launch time statistics in microseconds: .min, .max, .mean (src/pybind_api.cc:751-767)."""

    def __init__(self, results):
        self.min, self.max, self.mean = (float(v) for v in results)

    def __repr__(self):
        return "min_max_avg(us): %.2f %.2f %.2f" % (self.min, self.max, self.mean)


class Tester(PyKernel):
    __test__ = False  # not a pytest class

    def __init__(self, ker_type="", use_pass_opt=False, run_mode="dev"):
        PyKernel.__init__(self, ker_type, run_mode, int(os.getenv("DEVICE_ID") or 0))
        self._dynamic = "dyn" in ker_type
        self._generated = False
        self._expectations = []
        self._buffer_shape = {}  # strided stores: shape of the whole buffer behind the store
        del use_pass_opt  # the gfx950 pipeline is fixed; see set_passes

    # ---- random inputs the reference's tests draw through the harness (global NumPy generator, as there) ----
    @staticmethod
    def fast_random_normal(loc, scale, shape):
        """One random row repeated over every leading dim: cheap to make for large shapes."""
        out = np.empty(shape, np.float32)
        out[...] = np.random.normal(loc, scale, shape[-1])
        return out

    @staticmethod
    def bf16_random_normal(loc, scale, shape):
        """fp32 values that bf16 represents exactly (mantissa cut to 8 bits)."""
        bits = np.random.normal(loc, scale, shape).astype(np.float32).view(np.uint32)
        return ((bits >> 16) << 16).view(np.float32)

    # ---- inputs ----
    def _bound(self, make, array, dtype, offset=0):
        """A load made by make(host) and fed with `array`."""
        host = _host_array(array, dtype)
        op = make(host)
        self.input(op, host.data, offset)
        return op

    def load(self, shape_arr, dtype=None):
        if not isinstance(shape_arr, np.ndarray):  # a shape: the data arrives later through input()
            return PyKernel.load(self, shape_arr, as_datatype(dtype))
        return self._bound(lambda h: PyKernel.load(self, h.shape, h.dtype), shape_arr, dtype)

    def view_load(self, shape, stride, arr_dtype, offset=0, real_dtype=None):
        """The array is the whole buffer; the load reads `shape` elements of it through `stride` from `offset`."""
        if not isinstance(arr_dtype, np.ndarray):
            return PyKernel.view_load(self, shape, stride, as_datatype(arr_dtype))
        return self._bound(lambda h: PyKernel.view_load(self, shape, stride, h.dtype), arr_dtype, real_dtype, offset)

    def global_access(self, shape_arr, dtype=None):
        dtype = DataType.int32 if dtype is None else dtype
        if not isinstance(shape_arr, np.ndarray):
            return PyKernel.global_access(self, shape_arr, as_datatype(dtype))
        return self._bound(lambda h: PyKernel.global_access(self, h.shape, h.dtype), shape_arr, dtype)

    def gather_load(self, data_arr, index_op, axis=0, dtype=None, gather_mode=0):
        if not isinstance(data_arr, np.ndarray):
            return PyKernel.gather_load(self, data_arr, index_op, as_datatype(dtype), axis, gather_mode)
        return self._bound(lambda h: PyKernel.gather_load(self, h.shape, index_op, h.dtype, axis, gather_mode), data_arr, dtype)

    def one_hot(self, indices, depth, axis, on_value, off_value, dtype):
        return PyKernel.one_hot(self, indices, depth, axis, on_value, off_value, as_datatype(dtype))

    def slice_load(self, shape_arr, start, size, dtype=None):
        if not isinstance(shape_arr, np.ndarray):
            return PyKernel.slice_load(self, shape_arr, start, size, as_datatype(dtype))
        return self._bound(lambda h: PyKernel.slice_load(self, h.shape, start, size, h.dtype), shape_arr, dtype)

    def stridedslice_load(self, shape_arr, start, end, step, dtype=None):
        if not isinstance(shape_arr, np.ndarray):
            return PyKernel.stridedslice_load(self, shape_arr, start, end, step, as_datatype(dtype))
        return self._bound(lambda h: PyKernel.stridedslice_load(self, h.shape, start, end, step, h.dtype), shape_arr, dtype)

    # ---- operators that take a dtype by name ----
    def cast(self, x, dtype):
        return PyKernel.cast(self, x, as_datatype(dtype))

    def full(self, scalar, shape, dtype=None):
        return PyKernel.full(self, scalar, shape, as_datatype(dtype))

    # ---- outputs and expectations ----
    def store_expect(self, x, e, eps=None):
        op = PyKernel.store(self, x)
        self._expectations.append(Expectation(op, e, eps))
        return op

    def view_store_expect(self, x, stride, e, eps=None):
        """Stores x through `stride` into a buffer shaped like e (zeros where nothing is written) and expects e."""
        e = np.asarray(e)
        op = PyKernel.view_store(self, x, stride, e.size)
        self._buffer_shape[op._h] = tuple(e.shape)
        self._expectations.append(Expectation(op, e, eps, tuple(e.shape)))
        return op

    def clear_store_memory(self, store):
        """RtKernelPy.clear_store_memory (src/pybind_api.cc:874-877 of the reference) zeroes an output before the run, for
        element_any, which there only stores a value that is not zero. Here element_any always stores its result, so
        there is nothing to clear."""
        del store

    def output(self, store, shape=None):
        return PyKernel.output(self, store, shape if shape is not None else self._buffer_shape.get(store._h))

    def _readable(self, store):
        """The output as NumPy can compare it (bf16 widened to fp32)."""
        out = self.output(store)
        return PyKernel.convert_from_bf16(out) if store.dtype() == DataType.bfloat16 else out

    def check(self, store, expect, eps=None, verbose=False):
        got = self._readable(store)
        ok = Expectation(store, expect, eps).holds(got)
        if verbose and not ok:
            for title, value in (("OUTPUT", got), ("EXPECT", expect)):
                print("********** %s **********\n%s" % (title, value), file=sys.stderr)
        return ok

    # ---- code generation and runs ----
    def dump_verbose(self):
        print("******* graph *******\n%s\n********* bytecode *********\n%s" % (self.dump(), self.das()))

    def codegen(self, verbose=False):
        """Generates code; a kernel of fixed shapes does so once, a dynamic one at every call."""
        if not self._generated:
            PyKernel.codegen(self)
            self._generated = not self._dynamic
        if verbose:
            self.dump_verbose()

    def bare_run(self):
        """Launch only: no code generation."""
        PyKernel.run(self)

    def run(self, verbose=False):
        self.codegen()
        self.bare_run()
        if verbose:
            self.dump_verbose()

    def run_check(self, verbose=False):
        self.run(verbose)
        return all(self.check(x.store, x.want, x.eps, verbose) for x in self._expectations)

    def run_perf(self):
        self.codegen()
        return PerformanceResult(self.perf())

    # The reference's graph passes by the names its tests select them with (src/pybind_api.cc:616-650). What each
    # one achieves either always happens here or has no counterpart on an accumulator machine:
    _ALWAYS_DONE = ("DeadCodeEliminate", "EliminateReshape", "EliminateDiamondView")  # liveness; reshapes are views
    _NO_COUNTERPART = ("PrintPeakLive", "ReorderStore", "ReorderLoad", "CompactPeakLiveness", "VectorDoubleBuffer",
                       "InsertRemovePad", "VfFusion")  # scheduling of tiles in a unified buffer

    def set_passes(self, *pass_names):
        """The reference lets a test pick graph passes by name (python/dvm/tester.py:364-366). The pipeline here is
        fixed: the names are checked and remembered (`passes`), the generated code does not depend on them. A name the
        reference does not know is an error."""
        for name in pass_names:
            if name not in self._ALWAYS_DONE and name not in self._NO_COUNTERPART:
                raise RuntimeError("DVM EXCEPTION. reason: unknown pass '%s'" % name)
        self.passes = list(pass_names)

    def reset(self):
        PyKernel.reset(self)
        self._generated = False
        self._expectations = []
        self._buffer_shape = {}
