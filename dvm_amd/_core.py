"""ctypes binding of libdvm.so (include/dvm_c.h).

Mirrors the classes of the reference's pybind module `_dvm_py`
(include/dvm_py.h:277-388, src/pybind_api.cc:1066-1116): DataType, NDObject,
IntArrayRef, ScalarRef, Kernel (graph builder), PyKernel (builder + runner) and
Device, with the same method names and argument meaning.
"""
import ctypes
import os

import numpy as np

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
# DVM_HOST_LIBRARY names another build of the host library (the sanitizer build of `make asan=1`)
_LIB_PATH = os.environ.get("DVM_HOST_LIBRARY") or os.path.join(_LIB_DIR, "libdvm.so")


class _Operand(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int), ("obj", ctypes.c_void_p), ("ref", ctypes.c_void_p),
                ("f", ctypes.c_double), ("i", ctypes.c_int64)]


def _load():
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            "dvm_amd native library missing (%s): run `python -m dvm_amd.build` first" % _LIB_PATH)
    lib = ctypes.CDLL(_LIB_PATH)
    if not hasattr(lib, "dvm_rt_perf_samples"):
        raise ImportError("dvm_amd native library (%s) is older than the package: run `python -m dvm_amd.build`"
                          % _LIB_PATH)
    vp, ci, cs = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    i64p = ctypes.POINTER(ctypes.c_int64)
    opp = ctypes.POINTER(_Operand)
    sig = {
        "dvm_c_last_error": (ctypes.c_char_p, []),
        "dvm_rt_new": (vp, [ctypes.c_char_p, ctypes.c_char_p, ci]),
        "dvm_rt_delete": (None, [vp]),
        "dvm_rt_reset": (ci, [vp]),
        "dvm_rt_new_shape": (vp, [vp, i64p, cs]),
        "dvm_shape_update": (ci, [vp, i64p, cs]),
        "dvm_rt_new_scalar": (vp, [vp, ci]),
        "dvm_scalar_update_f": (ci, [vp, ctypes.c_double]),
        "dvm_scalar_update_i": (ci, [vp, ctypes.c_int64]),
        "dvm_rt_load": (vp, [vp, vp, ci]),
        "dvm_rt_store": (vp, [vp, vp]),
        "dvm_rt_unary": (vp, [vp, ci, vp]),
        "dvm_rt_binary": (vp, [vp, ci, opp, opp]),
        "dvm_rt_select": (vp, [vp, vp, vp, vp]),
        "dvm_rt_cast": (vp, [vp, vp, ci]),
        "dvm_rt_broadcast": (vp, [vp, vp, vp]),
        "dvm_rt_full": (vp, [vp, opp, vp, ci]),
        "dvm_rt_reshape": (vp, [vp, vp, vp]),
        "dvm_rt_reduce": (vp, [vp, ci, vp, vp, ci]),
        "dvm_rt_copy": (vp, [vp, vp]),
        "dvm_rt_matmul": (vp, [vp, vp, vp, ci, ci, vp]),
        "dvm_rt_set_store_inplace": (ci, [vp, vp]),
        "dvm_rt_set_store_temp": (ci, [vp, vp]),
        "dvm_rt_set_load_bind": (ci, [vp, vp, vp]),
        "dvm_rt_spec_next": (ci, [vp]),
        "dvm_rt_view_load": (vp, [vp, vp, vp, ci]),
        "dvm_rt_slice_load": (vp, [vp, vp, vp, vp, ci]),
        "dvm_rt_stridedslice_load": (vp, [vp, vp, vp, vp, vp, ci]),
        "dvm_rt_view_store": (vp, [vp, vp, vp, cs]),
        "dvm_obj_set_view_offset": (ci, [vp, ctypes.c_longlong]),
        "dvm_rt_permute": (vp, [vp, vp, vp]),
        "dvm_rt_global_access": (vp, [vp, vp, ci]),
        "dvm_rt_gather_load": (vp, [vp, vp, vp, ci, ci, ci]),
        "dvm_rt_pad_store": (vp, [vp, vp, ctypes.c_longlong]),
        "dvm_rt_one_hot": (vp, [vp, vp, vp, ci, ctypes.c_double, ctypes.c_double, ci]),
        "dvm_rt_element_any": (vp, [vp, vp]),
        "dvm_rt_grouped_matmul": (vp, [vp, vp, vp, ci, ci, vp, vp, ci, ci]),
        "dvm_rt_slice": (vp, [vp, vp, vp, vp]),
        "dvm_rt_slice_dim": (vp, [vp, vp, ci, vp, vp]),
        "dvm_rt_split": (ci, [vp, vp, ci, ctypes.c_longlong, cs, ctypes.POINTER(vp)]),
        "dvm_rt_concat": (vp, [vp, ctypes.POINTER(vp), cs, ci]),
        "dvm_rt_clone": (ci, [vp, vp, ctypes.POINTER(ci), ctypes.POINTER(vp), cs, ctypes.POINTER(vp)]),
        "dvm_rt_seq_add": (ci, [vp, ci, ctypes.c_uint]),
        "dvm_rt_parallel_add": (ci, [vp, ci, ctypes.c_uint, cs]),
        "dvm_obj_rank": (ci, [vp]),
        "dvm_obj_shape": (ci, [vp, i64p, cs]),
        "dvm_obj_dtype": (ci, [vp]),
        "dvm_rt_input": (ci, [vp, vp, vp, cs]),
        "dvm_rt_bind_device": (ci, [vp, vp, vp]),
        "dvm_rt_bind_device_view": (ci, [vp, vp, vp, i64p, cs]),
        "dvm_rt_set_workspace_allocator": (ci, [vp, vp, vp]),
        "dvm_rt_unbind_device": (ci, [vp]),
        "dvm_rt_normalize": (ci, [vp]),
        "dvm_rt_codegen": (ci, [vp]),
        "dvm_rt_jit_us": (ctypes.c_double, [vp]),
        "dvm_rt_run": (ci, [vp, vp, ci]),
        "dvm_rt_output": (ci, [vp, vp, vp, cs]),
        "dvm_rt_device_ptr": (vp, [vp, vp]),
        "dvm_rt_perf": (ci, [vp, ci, ci, ctypes.POINTER(ctypes.c_double)]),
        "dvm_rt_perf_samples": (ci, [vp, ci, ci, ctypes.POINTER(ctypes.c_double)]),
        "dvm_set_online_tuner": (None, [ci]),
        "dvm_set_lazy_tuner": (None, [ci]),
        "dvm_tuner_stats": (None, [ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64)]),
        "dvm_tuner_clear": (None, []),
        "dvm_rt_num_launches": (ci, [vp]),
        "dvm_rt_workspace_bytes": (cs, [vp]),
        "dvm_rt_program_count": (ci, [vp]),
        "dvm_rt_program": (ci, [vp, ci, vp, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32), cs]),
        "dvm_rt_das": (ctypes.c_char_p, [vp]),
        "dvm_rt_dump": (ctypes.c_char_p, [vp]),
        "dvm_rt_dump_r": (ctypes.c_char_p, [vp]),
        "dvm_rt_inspect": (ctypes.c_char_p, [vp]),
        "dvm_c_f32_to_bf16": (None, [vp, vp, cs]),
        "dvm_c_bf16_to_f32": (None, [vp, vp, cs]),
        "dvm_c_has_device": (ci, []),
        "dvm_c_core_num": (ci, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


class _LazyLib:
    """Loads libdvm.so at the first call, so that importing the package (the build step does) needs no
    built library; any use of the backend without one raises ImportError."""

    def __getattr__(self, name):
        lib = self.__dict__.get("_real")
        if lib is None:
            lib = self.__dict__["_real"] = _load()
            global _lib
            _lib = lib
        return getattr(lib, name)


_lib = _LazyLib()


def _check(ret):
    if ret is None or (isinstance(ret, int) and ret != 0 and not isinstance(ret, bool)):
        raise RuntimeError(_lib.dvm_c_last_error().decode())
    return ret


def _ptr(ret):
    if not ret:
        raise RuntimeError(_lib.dvm_c_last_error().decode())
    return ret


class DataType(int):
    """Element types; values match dvm::DataType (include/dvm.h)."""
    _names = {0: "bool", 1: "float16", 2: "bfloat16", 3: "float32", 4: "int32", 5: "int64"}

    def __repr__(self):
        return "DataType." + self._names.get(int(self), str(int(self)))

    __str__ = __repr__


DataType.bool = DataType(0)
DataType.float16 = DataType(1)
DataType.bfloat16 = DataType(2)
DataType.float32 = DataType(3)
DataType.int32 = DataType(4)
DataType.int64 = DataType(5)

_NP_OF = {0: np.bool_, 1: np.float16, 2: np.uint16, 3: np.float32, 4: np.int32, 5: np.int64}
_ITEMSIZE = {0: 1, 1: 2, 2: 2, 3: 4, 4: 4, 5: 8}


def _i64(seq):
    arr = (ctypes.c_int64 * max(1, len(seq)))(*[int(v) for v in seq])
    return arr, len(seq)


class NDObject:
    def __init__(self, handle):
        self._h = handle

    def shape(self):
        buf = (ctypes.c_int64 * 10)()
        r = _lib.dvm_obj_shape(self._h, buf, 10)
        return tuple(buf[i] for i in range(r))

    def dtype(self):
        return DataType(_lib.dvm_obj_dtype(self._h))


class IntArrayRef:
    """A shape (or axis list) whose values can change between codegen calls."""

    def __init__(self, rt, shape=(), handle=None):
        if handle is not None:  # an existing reference of a cloned kernel
            self._h = handle
        else:
            arr, n = _i64(shape)
            self._h = _ptr(_lib.dvm_rt_new_shape(rt, arr, n))
        self._shape = tuple(int(v) for v in shape)

    def shape(self):
        return self._shape

    def update(self, shape):
        arr, n = _i64(shape)
        _lib.dvm_shape_update(self._h, arr, n)
        self._shape = tuple(int(v) for v in shape)


class ScalarRef:
    """A scalar whose value is read again at every codegen."""

    def __init__(self, rt, dtype, handle=None):
        self._h = handle if handle is not None else _ptr(_lib.dvm_rt_new_scalar(rt, int(dtype)))

    def update(self, value):
        if isinstance(value, (int, np.integer)) and not isinstance(value, bool):
            _lib.dvm_scalar_update_i(self._h, int(value))
        else:
            _lib.dvm_scalar_update_f(self._h, float(value))


_UNARY = ["sqrt", "abs", "log", "exp", "reciprocal", "isfinite", "logical_not", "round", "floor", "ceil", "trunc"]
_BINARY = ["equal", "not_equal", "greater", "greater_equal", "less", "less_equal", "add", "sub", "mul", "div", "pow",
           "maximum", "minimum", "logical_and", "logical_or"]


class Kernel:
    """Graph builder; method names follow include/dvm_py.h:301-387."""

    K_VEC, K_CUBE, K_MIX, K_PARAL, K_SEQ, K_SPLIT, K_EAGER = range(7)
    F_DYN, F_UWS, F_SPEC = 1, 2, 4

    def __init__(self):
        self._rt = None
        self._keep = []
        self._pad_of = {}  # pad_store handle -> pad size

    # -- references --
    def _shape_ref(self, shape):
        if isinstance(shape, IntArrayRef):
            return shape
        ref = IntArrayRef(self._rt, list(shape))
        self._keep.append(ref)
        return ref

    def int_array(self):
        ref = IntArrayRef(self._rt, [])
        self._keep.append(ref)
        return ref

    def scalar(self, dtype=DataType.float32):
        ref = ScalarRef(self._rt, dtype)
        self._keep.append(ref)
        return ref

    def _operand(self, v):
        o = _Operand()
        if isinstance(v, NDObject):
            o.kind, o.obj = 0, v._h
        elif isinstance(v, ScalarRef):
            o.kind, o.ref = 3, v._h
        elif isinstance(v, (bool, np.bool_)):
            o.kind, o.i = 2, int(v)
        elif isinstance(v, (int, np.integer)):
            o.kind, o.i = 2, int(v)
        elif isinstance(v, (float, np.floating)):
            o.kind, o.f = 1, float(v)
        else:
            raise TypeError("unsupported operand: %r" % (v,))
        return o

    def _wrap(self, h):
        return NDObject(_ptr(h))

    # -- tensor access --
    def load(self, shape, type):
        return self._wrap(_lib.dvm_rt_load(self._rt, self._shape_ref(shape)._h, int(type)))

    def store(self, obj, type=None):
        if type is not None and int(type) != int(obj.dtype()):
            obj = self.cast(obj, type)
        return self._wrap(_lib.dvm_rt_store(self._rt, obj._h))

    def set_store_inplace(self, store):
        _check(_lib.dvm_rt_set_store_inplace(self._rt, store._h))

    def set_store_temp(self, store):
        """The store is no output of the kernel, only what loads bound to it read (KernelPy.set_store_temp)."""
        _check(_lib.dvm_rt_set_store_temp(self._rt, store._h))

    def set_load_bind(self, load, store):
        """The load reads what `store` (a store of this kernel) writes; call it before the load's first use."""
        _check(_lib.dvm_rt_set_load_bind(self._rt, load._h, store._h))

    def spec_next(self):
        """Stage marker of a kernel created as "vector:spec" (RtKernelPy.spec_next)."""
        _check(_lib.dvm_rt_spec_next(self._rt))

    # -- strided views (include/dvm_py.h view_load / slice_load / stridedslice_load); innermost stride 1 --
    def view_load(self, shape, stride, type):
        return self._wrap(_lib.dvm_rt_view_load(self._rt, self._shape_ref(shape)._h, self._shape_ref(stride)._h, int(type)))

    def slice_load(self, shape, start, size, type):
        return self._wrap(_lib.dvm_rt_slice_load(self._rt, self._shape_ref(shape)._h, self._shape_ref(start)._h,
                                                 self._shape_ref(size)._h, int(type)))

    def stridedslice_load(self, shape, start, end, step, type):
        return self._wrap(_lib.dvm_rt_stridedslice_load(self._rt, self._shape_ref(shape)._h, self._shape_ref(start)._h,
                                                        self._shape_ref(end)._h, self._shape_ref(step)._h, int(type)))

    def view_store(self, obj, stride, extent):
        """Stores obj through element strides into a zero-initialised buffer of `extent` elements."""
        return self._wrap(_lib.dvm_rt_view_store(self._rt, obj._h, self._shape_ref(stride)._h, int(extent)))

    # -- gathers, one-hot, padded stores (include/dvm_py.h:302-327 of the reference) --
    def global_access(self, shape, type):
        """Names a tensor for another operator to read (the int32 index of gather_load); fed like a load."""
        return self._wrap(_lib.dvm_rt_global_access(self._rt, self._shape_ref(shape)._h, int(type)))

    def gather_load(self, shape, index, type, axis=0, gather_mode=0):
        """The tensor of `shape` fed to the returned operator, read at `index` along `axis`: gather_mode 0 is NumPy's
        take_along_axis, 1 its take. Negative indices count from the end; indices past either end are clipped."""
        return self._wrap(_lib.dvm_rt_gather_load(self._rt, self._shape_ref(shape)._h, index._h, int(type), int(axis), int(gather_mode)))

    def pad_store(self, obj, pad_size):
        """Stores obj into a buffer whose innermost rows are pad_size elements longer (zeros there); output() gives
        that whole buffer."""
        op = self._wrap(_lib.dvm_rt_pad_store(self._rt, obj._h, int(pad_size)))
        self._pad_of[op._h] = int(pad_size)
        return op

    def one_hot(self, indices, depth, axis, on_value, off_value, type):
        """A dim of extent depth at position axis: on_value where the position equals the int32 index, else off_value."""
        depth_ref = depth if isinstance(depth, IntArrayRef) else self._shape_ref([int(depth)])
        return self._wrap(_lib.dvm_rt_one_hot(self._rt, indices._h, depth_ref._h, int(axis), float(on_value), float(off_value), int(type)))

    def element_any(self, input):
        """One fp32 value: the maximum over every element (1 when any element of a 0 / 1 mask is set)."""
        return self._wrap(_lib.dvm_rt_element_any(self._rt, input._h))

    # -- views of values (include/dvm_py.h:163-189 of the reference): nothing is copied --
    def permute(self, input, dims):
        return self._wrap(_lib.dvm_rt_permute(self._rt, input._h, self._shape_ref(dims)._h))

    def slice(self, input, start, size):
        return self._wrap(_lib.dvm_rt_slice(self._rt, input._h, self._shape_ref(start)._h, self._shape_ref(size)._h))

    def _int_scalar(self, v):
        if isinstance(v, ScalarRef):
            return v
        ref = self.scalar(DataType.int32)
        ref.update(int(v))
        return ref

    def slice_dim(self, input, dim, begin, end):
        return self._wrap(_lib.dvm_rt_slice_dim(self._rt, input._h, int(dim), self._int_scalar(begin)._h, self._int_scalar(end)._h))

    def concat(self, inputs, dim):
        arr = (ctypes.c_void_p * len(inputs))(*[x._h for x in inputs])
        return self._wrap(_lib.dvm_rt_concat(self._rt, arr, len(inputs), int(dim)))

    def split(self, input, dim, split_size, split_num):
        out = (ctypes.c_void_p * int(split_num))()
        _check(_lib.dvm_rt_split(self._rt, input._h, int(dim), int(split_size), int(split_num), out))
        return tuple(self._wrap(out[i]) for i in range(int(split_num)))

    # -- sub-kernel groups of "seq" / "parallel" kernels (include/dvm_py.h:369-371) --
    def seq_add(self, ktype, flags=0):
        _check(_lib.dvm_rt_seq_add(self._rt, int(ktype), int(flags)))

    def parallel_add(self, ktype, flags=0, core_limit=0):
        _check(_lib.dvm_rt_parallel_add(self._rt, int(ktype), int(flags), int(core_limit)))

    # -- operators --
    def cast(self, input, type):
        return self._wrap(_lib.dvm_rt_cast(self._rt, input._h, int(type)))

    def select(self, cond, lhs, rhs):
        return self._wrap(_lib.dvm_rt_select(self._rt, cond._h, lhs._h, rhs._h))

    def broadcast(self, input, shape):
        return self._wrap(_lib.dvm_rt_broadcast(self._rt, input._h, self._shape_ref(shape)._h))

    def full(self, scalar, shape, dtype):
        op = self._operand(scalar)
        return self._wrap(_lib.dvm_rt_full(self._rt, ctypes.byref(op), self._shape_ref(shape)._h, int(dtype)))

    def reshape(self, input, shape):
        return self._wrap(_lib.dvm_rt_reshape(self._rt, input._h, self._shape_ref(shape)._h))

    def copy(self, input):
        return self._wrap(_lib.dvm_rt_copy(self._rt, input._h))

    def _reduce(self, kind, input, dims, keepdims):
        if isinstance(dims, int):
            dims = (dims,)
        return self._wrap(_lib.dvm_rt_reduce(self._rt, kind, input._h, self._shape_ref(dims)._h, int(bool(keepdims))))

    def sum(self, input, dims, keepdims=False):
        return self._reduce(0, input, dims, keepdims)

    def max(self, input, dims, keepdims=False):
        return self._reduce(1, input, dims, keepdims)

    def min(self, input, dims, keepdims=False):
        return self._reduce(2, input, dims, keepdims)

    def matmul(self, lhs, rhs, trans_a, trans_b, bias=None):
        return self._wrap(_lib.dvm_rt_matmul(self._rt, lhs._h, rhs._h, int(bool(trans_a)), int(bool(trans_b)),
                                             bias._h if bias is not None else None))

    def grouped_matmul(self, lhs, rhs, trans_a, trans_b, bias, group_list, group_type, group_list_type=0):
        """One product per group (KernelPy.grouped_matmul). group_type 0: the groups are ranges of lhs's rows, rhs is
        [groups, k, n], the result [m, n]; 2: ranges of the k axis, the result [groups, m, n]. group_list: a load of
        int64 values, the ranges' upper bounds (group_list_type 0) or sizes (1), read on the device at every launch."""
        return self._wrap(_lib.dvm_rt_grouped_matmul(self._rt, lhs._h, rhs._h, int(bool(trans_a)), int(bool(trans_b)),
                                                     bias._h if bias is not None else None, group_list._h,
                                                     int(group_type), int(group_list_type)))

    # -- introspection --
    def das(self):
        return _ptr(_lib.dvm_rt_das(self._rt)).decode()

    def dump(self):
        return _ptr(_lib.dvm_rt_dump(self._rt)).decode()

    def dump_r(self):
        return _ptr(_lib.dvm_rt_dump_r(self._rt)).decode()

    def inspect(self):
        return _ptr(_lib.dvm_rt_inspect(self._rt)).decode()


def _make_unary(idx):
    def fn(self, input):
        return self._wrap(_lib.dvm_rt_unary(self._rt, idx, input._h))
    return fn


def _make_binary(idx):
    def fn(self, lhs, rhs):
        a, b = self._operand(lhs), self._operand(rhs)
        return self._wrap(_lib.dvm_rt_binary(self._rt, idx, ctypes.byref(a), ctypes.byref(b)))
    return fn


for _i, _n in enumerate(_UNARY):
    setattr(Kernel, _n, _make_unary(_i))
for _i, _n in enumerate(_BINARY):
    setattr(Kernel, _n, _make_binary(_i))


class PyKernel(Kernel):
    """Builder plus runner: owns device buffers for the bound numpy inputs and the outputs."""

    def __init__(self, ker_type, run_type, dev_id):
        Kernel.__init__(self)
        self._rt = _ptr(_lib.dvm_rt_new(ker_type.encode(), run_type.encode(), int(dev_id)))
        self._run_type = run_type
        self._dyn = "dyn" in ker_type
        self._load_shape = {}   # load handle -> IntArrayRef
        self._inputs = {}

    def __del__(self):
        rt, self._rt = getattr(self, "_rt", None), None
        if rt:
            _lib.dvm_rt_delete(rt)

    def load(self, shape, type):
        ref = self._shape_ref(shape)
        op = Kernel.load(self, ref, type)
        self._load_shape[op._h] = ref
        return op

    def global_access(self, shape, type):
        ref = self._shape_ref(shape)
        op = Kernel.global_access(self, ref, type)
        self._load_shape[op._h] = ref
        return op

    def gather_load(self, shape, index, type, axis=0, gather_mode=0):
        ref = self._shape_ref(shape)  # the source tensor's shape: input() on the returned operator updates it
        op = Kernel.gather_load(self, ref, index, type, axis, gather_mode)
        self._load_shape[op._h] = ref
        return op

    def load_shape(self, load):
        """The updatable shape behind a load (update it and generate code again to change the extent)."""
        return self._load_shape[load._h]

    def clone(self, base, remap):
        """Copies `base`'s graph into this kernel (RtKernelPy::Clone, src/pybind_api.cc:923-993). `remap` lists
        operators, shape / axis references and scalar references of `base`; their counterparts here are returned."""
        items = list(remap)
        base_loads = list(base._load_shape.items())  # (load handle, IntArrayRef)
        kinds, handles = [], []
        for it in items:
            kinds.append(1 if isinstance(it, IntArrayRef) else (2 if isinstance(it, ScalarRef) else 0))
            handles.append(it._h)
        for h, ref in base_loads:
            kinds += [0, 1]
            handles += [h, ref._h]
        n = len(kinds)
        ck = (ctypes.c_int * n)(*kinds)
        ch = (ctypes.c_void_p * n)(*handles)
        co = (ctypes.c_void_p * n)()
        _check(_lib.dvm_rt_clone(self._rt, base._rt, ck, ch, n, co))
        self._keep, self._load_shape, self._inputs = [], {}, {}
        out = []
        for i, it in enumerate(items):
            if kinds[i] == 1:
                w = IntArrayRef(self._rt, it.shape(), handle=co[i])
            elif kinds[i] == 2:
                w = ScalarRef(self._rt, None, handle=co[i])
            else:
                w = self._wrap(co[i])
            self._keep.append(w)
            out.append(w)
        for j, (h, ref) in enumerate(base_loads):
            i = len(items) + 2 * j
            sref = IntArrayRef(self._rt, ref.shape(), handle=co[i + 1])
            self._keep.append(sref)
            self._load_shape[co[i]] = sref
        return tuple(out)

    def reset(self):
        _check(_lib.dvm_rt_reset(self._rt))
        self._keep = []
        self._pad_of = {}
        self._load_shape = {}
        self._inputs = {}

    @staticmethod
    def convert_to_bf16(array):
        src = np.asarray(array, dtype=np.float32, order="C")  # keeps rank 0, which ascontiguousarray would not
        dst = np.empty(src.shape, dtype=np.uint16)
        _lib.dvm_c_f32_to_bf16(src.ctypes.data, dst.ctypes.data, src.size)
        return dst

    @staticmethod
    def convert_from_bf16(array):
        src = np.asarray(array, dtype=np.uint16, order="C")
        dst = np.empty(src.shape, dtype=np.float32)
        _lib.dvm_c_bf16_to_f32(src.ctypes.data, dst.ctypes.data, src.size)
        return dst

    def input(self, load, array, offset=0):
        """Binds a numpy array (copied to the device), a scalar value, or a shape to a placeholder."""
        if isinstance(load, ScalarRef):
            load.update(array)
            return
        if isinstance(load, IntArrayRef):
            load.update(list(array))
            return
        arr = np.asarray(array, order="C")
        if offset:
            _check(_lib.dvm_obj_set_view_offset(load._h, int(offset)))
        ref = self._load_shape.get(load._h)
        if ref is not None and tuple(ref.shape()) != tuple(arr.shape):
            ref.update(list(arr.shape))
        want = _ITEMSIZE[int(load.dtype())]
        if arr.dtype.itemsize != want:
            raise TypeError("array dtype %s does not match the load's element size %d" % (arr.dtype, want))
        self._inputs[load._h] = arr
        _check(_lib.dvm_rt_input(self._rt, load._h, arr.ctypes.data, arr.nbytes))

    def bind_device(self, io, device_ptr, shape=None, strides=None):
        """Binds caller-owned device memory (e.g. a torch tensor's data_ptr()) to a load or store. `strides`
        (elements, one per dim) binds a load to memory that is not contiguous: it is then read through them."""
        if shape is not None and io._h in self._load_shape:
            self._load_shape[io._h].update(list(shape))
        if strides is not None:
            arr, n = _i64(strides)
            _check(_lib.dvm_rt_bind_device_view(self._rt, io._h, ctypes.c_void_p(device_ptr), arr, n))
        elif io._h in self._load_shape:  # (a load that was strided at an earlier call is dense again)
            _check(_lib.dvm_rt_bind_device_view(self._rt, io._h, ctypes.c_void_p(device_ptr), None, 0))
        else:
            _check(_lib.dvm_rt_bind_device(self._rt, io._h, ctypes.c_void_p(device_ptr)))

    def set_workspace_allocator(self, alloc):
        """`alloc(nbytes) -> device address` supplies the workspace of the launches from now on (a framework's
        caching allocator); None gives it back to the runner. The memory has to stay valid until the launches of
        the run that follows have finished."""
        if alloc is None:
            self._ws_callback = None
            _check(_lib.dvm_rt_set_workspace_allocator(self._rt, None, None))
            return
        proto = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p)
        self._ws_callback = proto(lambda nbytes, _user: int(alloc(int(nbytes))))  # kept alive with the kernel
        _check(_lib.dvm_rt_set_workspace_allocator(self._rt, ctypes.cast(self._ws_callback, ctypes.c_void_p), None))

    def normalize(self):
        """Shape inference only: store.shape() is valid afterwards."""
        _check(_lib.dvm_rt_normalize(self._rt))

    def release_device_bindings(self):
        """Forgets caller-owned device memory bound earlier; the next input() / codegen() use buffers of the runner."""
        _check(_lib.dvm_rt_unbind_device(self._rt))

    def codegen(self, pass_names=None):
        """Normalize + CodeGen. `pass_names` is the reference's argument (src/pybind_api.cc:616): the pipeline here is
        fixed and the generated code does not depend on it (Tester.set_passes checks the names).

        A dynamic kernel whose placeholder loads have no shape yet (negative dims, nothing bound) has nothing to
        generate code for: the call returns and the run that follows the inputs generates it. (The reference's
        graph kernel compiles symbolic shapes at this point, tests/ut/test_split_sym_graph.py:193-214.)"""
        if any(d < 0 for ref in self._load_shape.values() for d in ref.shape()):
            return
        _check(_lib.dvm_rt_codegen(self._rt))

    def jit_us(self):
        return _lib.dvm_rt_jit_us(self._rt)

    def run(self, stream=None, sync=True, on_given_stream=False):
        """Launches on the runner's own stream, or on `stream` (a hipStream_t as an integer). With on_given_stream
        the handle is taken as it is, 0 naming the device's default stream (what torch's default stream is)."""
        flags = (1 if sync else 0) | (2 if on_given_stream else 0)
        _check(_lib.dvm_rt_run(self._rt, ctypes.c_void_p(stream) if stream else None, flags))

    def output(self, store, shape=None):
        """The stored tensor; `shape` (strided stores) reads back the whole buffer the store wrote into."""
        shape = store.shape() if shape is None else tuple(shape)
        if store._h in self._pad_of and len(shape) > 0:
            shape = tuple(shape[:-1]) + (shape[-1] + self._pad_of[store._h],)
        dt = int(store.dtype())
        out = np.empty(shape, dtype=_NP_OF[dt])
        _check(_lib.dvm_rt_output(self._rt, store._h, out.ctypes.data, out.nbytes))
        return out

    def device_ptr(self, io):
        return _lib.dvm_rt_device_ptr(self._rt, io._h)

    def perf(self, warmup=3, iters=10):
        out = (ctypes.c_double * 3)()
        _check(_lib.dvm_rt_perf(self._rt, warmup, iters, out))
        return (out[0], out[1], out[2])

    def programs(self):
        """The compiled launches as (blob bytes, (workgroups, threads, lds_bytes), [workspace word indices]); the
        workspace words of a blob hold byte offsets into the workspace (include/dvm_c.h, dvm_rt_program)."""
        out = []
        for i in range(_lib.dvm_rt_program_count(self._rt)):
            blob = (ctypes.c_uint8 * 4096)()
            geo = (ctypes.c_uint32 * 3)()
            words = (ctypes.c_uint32 * 64)()
            n = _lib.dvm_rt_program(self._rt, i, blob, geo, words, 64)
            if n < 0:
                raise RuntimeError(_lib.dvm_c_last_error().decode())
            out.append((bytes(blob), (geo[0], geo[1], geo[2]), [words[j] for j in range(n)]))
        return out

    def perf_samples(self, warmup=3, iters=20):
        """Microseconds of each of `iters` launches (HIP events on the runner's stream), after `warmup` launches."""
        out = (ctypes.c_double * iters)()
        _check(_lib.dvm_rt_perf_samples(self._rt, warmup, iters, out))
        return [out[i] for i in range(iters)]

    def num_launches(self):
        return _lib.dvm_rt_num_launches(self._rt)

    def workspace_bytes(self):
        return _lib.dvm_rt_workspace_bytes(self._rt)

    @staticmethod
    def barrier():
        pass

    @staticmethod
    def set_deterministic(enable):
        """Config::SetDeterm of the reference picks ordered reduces over atomics. Reduces here never use atomics
        (one team of lanes owns an output and combines in a fixed order), so both settings give the same bits."""
        pass

    @staticmethod
    def set_online_tuning(enable):
        """Config::SetOnlineTuner of the reference (include/dvm.h:735): the first code generation of a matmul shape on
        a machine with a device times every (block tile, parts of the k axis) candidate there and remembers the
        fastest for the process; without it tile and split come from figures measured once on an MI355X."""
        _lib.dvm_set_online_tuner(1 if enable else 0)

    @staticmethod
    def set_lazy_tuning(enable):
        """Config::SetLazyTuner (include/dvm.h:737). The reference's lazy tuner spreads its trials over the launches
        of the application; a trial here costs microseconds to compile, so both switches tune at the first code
        generation of a shape."""
        _lib.dvm_set_lazy_tuner(1 if enable else 0)

    @staticmethod
    def tuner_stats():
        """(product shapes measured so far, entries of the tuner's table)."""
        a, b = ctypes.c_uint64(0), ctypes.c_uint64(0)
        _lib.dvm_tuner_stats(ctypes.byref(a), ctypes.byref(b))
        return int(a.value), int(b.value)

    @staticmethod
    def tuner_clear():
        _lib.dvm_tuner_clear()

    def tile(self, start, end, num, factor=0):
        """Manual tiling of the reference's tile model (RtKernelPy::Tile, src/pybind_api.cc:1093). The gfx950
        schedules have no user-visible tiles; the hint is accepted and ignored."""
        pass


class Device:
    @staticmethod
    def arch():
        return "gfx950"

    @staticmethod
    def core_num():
        return _lib.dvm_c_core_num()

    @staticmethod
    def soc_name():
        return "MI355X"

    @staticmethod
    def available():
        return bool(_lib.dvm_c_has_device())
