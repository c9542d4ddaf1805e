"""CPU oracle for the DVM path: eager evaluation of a DVM graph. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the product package dvm_amd never does.

`OracleKernel` offers the same builder methods as the product's Tester / PyKernel
(load, add, sum, cast, select, matmul, store ...), but computes every operator at
once on the CPU with the scalar C functors of oracle/dvm_oracle.c. The dtype
lowering rules are restated here from the reference, independently of the
product's C++:
  * bool operands compute as fp16 and convert back (src/dvm.cc:445-460,1245-1283,1298-1324);
  * bf16 unary ops, bf16 div/pow and fp16 pow / round..trunc compute in fp32 (src/dvm.cc:1252-1258,1326-1337);
  * reciprocal(x) = 1 / x, logical_not(x) = 1 - x (src/dvm.cc:1272-1279);
  * x - s = x + (-s), s - x = x * (-1) + s (src/dvm.cc:663-673);
  * pow(x, integer) = repeated squaring (+ reciprocal) (src/dvm.cc:255-279), pow(s > 0, x) = exp(x * ln s) (:652-660);
  * compares produce 1/0 in the operand type, then convert to bool through fp16 (src/dvm.cc:1372-1375,425-443);
  * casts go through the intermediate types of the routing table (src/dvm.cc:416-423,1429-1447);
  * sum needs fp32 input (src/dvm.cc:1537-1540) and accumulates in fp64 (src/vm_gpu.cu:779-866).
Values are numpy arrays: bool_ for bool, int32 for int32, float32 holding
fp16- / bf16- / fp32-representable numbers for the float types.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "libdvm_oracle.so")

BOOL, F16, BF16, F32, I32, I64 = 0, 1, 2, 3, 4, 5
_NAMES = {"bool": BOOL, "float16": F16, "bfloat16": BF16, "float32": F32, "int32": I32, "int64": I64}

SQRT, ABS, LOG, EXP, RECIP, ISFINITE, LNOT, ROUND, FLOOR, CEIL, TRUNC = range(11)
EQ, NE, GT, GE, LT, LE, ADD, SUB, MUL, DIV, POW, MAXIMUM, MINIMUM, LAND, LOR = range(15)


def build():
    """Compiles oracle/dvm_oracle.c (gcc) if the shared object is missing or stale."""
    src = os.path.join(_DIR, "dvm_oracle.c")
    if not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _DIR, "-B", "libdvm_oracle.so"], check=True, capture_output=True)
    return _SO


def _lib():
    global _LIB
    try:
        return _LIB
    except NameError:
        pass
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    lib.ora_f16_to_f32.restype = ctypes.c_float
    lib.ora_f16_to_f32.argtypes = [ctypes.c_uint16]
    lib.ora_f32_to_f16.restype = ctypes.c_uint16
    lib.ora_f32_to_f16.argtypes = [ctypes.c_float]
    lib.ora_bf16_to_f32.restype = ctypes.c_float
    lib.ora_bf16_to_f32.argtypes = [ctypes.c_uint16]
    lib.ora_f32_to_bf16_dev.restype = ctypes.c_uint16
    lib.ora_f32_to_bf16_dev.argtypes = [ctypes.c_float]
    lib.ora_f32_to_bf16_host.restype = ctypes.c_uint16
    lib.ora_f32_to_bf16_host.argtypes = [ctypes.c_float]
    _LIB = lib
    return lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dt):
    return np.asarray(a, dtype=dt, order="C")  # a value of rank 0 keeps its rank (src/ops.cc:3080-3117 reduces to rank 0)


# ---- raw functors on arrays ---------------------------------------------------------

def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    _lib().ora_f32_to_f16_bits(_p(x), _p(out), ctypes.c_size_t(x.size))
    return out


def f16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    _lib().ora_f16_bits_to_f32(_p(h), _p(out), ctypes.c_size_t(h.size))
    return out


def f32_to_bf16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    _lib().ora_f32_to_bf16_bits(_p(x), _p(out), ctypes.c_size_t(x.size))
    return out


def bf16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    _lib().ora_bf16_bits_to_f32(_p(h), _p(out), ctypes.c_size_t(h.size))
    return out


def round_to(t, x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.float32)
    _lib().ora_round_f(t, _p(x), _p(out), ctypes.c_size_t(x.size))
    return out


def unary_f(op, t, x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.float32)
    _lib().ora_unary_f(op, t, _p(x), _p(out), ctypes.c_size_t(x.size))
    return out


def binary_f(op, t, a, b):
    a, b = np.broadcast_arrays(a, b)
    a, b = _c(a, np.float32), _c(b, np.float32)
    out = np.empty(a.shape, np.float32)
    _lib().ora_binary_f(op, t, _p(a), _p(b), _p(out), ctypes.c_size_t(a.size))
    return out


def binary_i32(op, a, b):
    a, b = np.broadcast_arrays(a, b)
    a, b = _c(a, np.int32), _c(b, np.int32)
    out = np.empty(a.shape, np.int32)
    _lib().ora_binary_i32(op, _p(a), _p(b), _p(out), ctypes.c_size_t(a.size))
    return out


def compare(op, a, b, is_int):
    a, b = np.broadcast_arrays(a, b)
    if is_int:
        a, b = _c(a, np.int32), _c(b, np.int32)
        out = np.empty(a.shape, np.int32)
        _lib().ora_compare_i32(op, _p(a), _p(b), _p(out), ctypes.c_size_t(a.size))
    else:
        a, b = _c(a, np.float32), _c(b, np.float32)
        out = np.empty(a.shape, np.float32)
        _lib().ora_compare_f(op, _p(a), _p(b), _p(out), ctypes.c_size_t(a.size))
    return out


def reduce_f32(kind, x, axes, keepdims):
    """Reduces x (float32) over `axes` one axis at a time, fp64 accumulation per axis for sums."""
    x = _c(x, np.float32)
    axes = sorted(a % x.ndim for a in axes)
    # move the reduced axes together so that a sum accumulates over all of them in fp64 at once
    kept = [a for a in range(x.ndim) if a not in axes]
    xt = np.ascontiguousarray(np.transpose(x, kept + axes))
    outer = int(np.prod([x.shape[a] for a in kept], dtype=np.int64)) if kept else 1
    red = int(np.prod([x.shape[a] for a in axes], dtype=np.int64)) if axes else 1
    out = np.empty((outer,), np.float32)
    _lib().ora_reduce_f32(kind, _p(xt), ctypes.c_size_t(outer), ctypes.c_size_t(red), ctypes.c_size_t(1), _p(out))
    shape = [x.shape[a] for a in kept]
    out = out.reshape(shape)
    if keepdims:
        full = [1 if a in axes else x.shape[a] for a in range(x.ndim)]
        out = out.reshape(full)
    return out


def matmul(a, b, bias, trans_a, trans_b, t):
    a, b = _c(a, np.float32), _c(b, np.float32)
    m = a.shape[-1] if trans_a else a.shape[-2]
    k = a.shape[-2] if trans_a else a.shape[-1]
    n = b.shape[-2] if trans_b else b.shape[-1]
    batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    nb = int(np.prod(batch, dtype=np.int64))  # (spelled out: a -1 cannot be inferred next to an empty matrix)
    ab = np.broadcast_to(a, batch + a.shape[-2:]).reshape((nb,) + a.shape[-2:])
    bb = np.broadcast_to(b, batch + b.shape[-2:]).reshape((nb,) + b.shape[-2:])
    out = np.empty((nb, m, n), np.float32)
    bias_c = _c(bias, np.float32) if bias is not None else None
    for i in range(ab.shape[0]):
        ai, bi, oi = np.ascontiguousarray(ab[i]), np.ascontiguousarray(bb[i]), out[i]
        _lib().ora_matmul(_p(ai), _p(bi), _p(bias_c) if bias_c is not None else None, _p(oi), ctypes.c_size_t(m),
                          ctypes.c_size_t(n), ctypes.c_size_t(k), int(trans_a), int(trans_b), t)
    return out.reshape(batch + (m, n))


def batchnorm_nchw(x, gamma, beta, eps):
    x = _c(x, np.float32)
    n, c = x.shape[0], x.shape[1]
    hw = int(np.prod(x.shape[2:], dtype=np.int64))
    y = np.empty_like(x)
    g, b = _c(gamma, np.float32).reshape(-1), _c(beta, np.float32).reshape(-1)
    _lib().ora_batchnorm_nchw(_p(x), _p(g), _p(b), _p(y), ctypes.c_size_t(n), ctypes.c_size_t(c), ctypes.c_size_t(hw),
                              ctypes.c_float(eps))
    return y


# ---- graph evaluator ------------------------------------------------------------------

class OVal:
    """A value of the graph: numpy array + DVM element type + whether it came out of a compare / logical op."""

    def __init__(self, a, t, bool_result=False, is_load=False):
        self.a = a
        self.t = t
        self.bool_result = bool_result
        self.is_load = is_load

    def shape(self):
        return tuple(self.a.shape)

    def dtype(self):
        return self.t


# intermediate type of one conversion step (row = from, column = to), src/dvm.cc:416-423
_ROUTE = {
    BOOL: {F16: F16, BF16: F16, F32: F16, I32: F16},
    F16: {BOOL: BOOL, BF16: F32, F32: F32, I32: I32},
    BF16: {BOOL: F32, F16: F32, F32: F32, I32: I32},
    F32: {BOOL: F16, F16: F16, BF16: BF16, I32: I32},
    I32: {BOOL: F16, F16: F16, BF16: F32, F32: F32},
}


def _tid(dtype):
    if isinstance(dtype, str):
        return _NAMES[dtype]
    return int(dtype)


class OracleKernel:
    K_VEC, K_CUBE, K_MIX = 0, 1, 2

    def __init__(self):
        self.stores = []

    # Group markers of sequence / parallel kernels (include/dvm.h:250-251 of the reference) say where
    # launches end, not what is computed: the restatement evaluates operator by operator either way.
    def seq_add(self, ktype, flags=0):
        pass

    def parallel_add(self, ktype, flags=0, core_limit=0):
        pass

    # -- leaves --
    def load(self, array, dtype=None):
        a = np.asarray(array)
        t = _tid(dtype) if dtype is not None else _NAMES[str(a.dtype)]
        if t == I64:  # carried as it is: only the group list of a grouped matmul has this type here
            v = a.astype(np.int64)
        elif t == BOOL:
            v = a.astype(np.bool_)
        elif t == I32:
            v = a.astype(np.int32)
        elif t == F16:
            v = a.astype(np.float16).astype(np.float32)
        elif t == BF16:
            v = bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32)))
        else:
            v = a.astype(np.float32)
        return OVal(v, t, is_load=True)

    # Views (include/dvm.h:294,312,317,339 of the reference): a load reads element i0..in of its shape at
    # offset + sum(i_d * stride_d) of the flat buffer; slice loads are the NumPy basic slices of the same
    # bounds (negative bounds count from the end, bounds past the end are clipped); a strided store writes
    # element i0..in of its value at sum(i_d * stride_d) of a zero-filled flat buffer.
    def view_load(self, shape, stride, array, offset=0, real_dtype=None):
        flat = np.ascontiguousarray(array).reshape(-1)
        idx = np.full(tuple(shape), int(offset), np.int64)
        for d, (n, st) in enumerate(zip(shape, stride)):
            ext = [1] * len(shape)
            ext[d] = n
            idx = idx + (np.arange(n, dtype=np.int64) * int(st)).reshape(ext)
        return self.load(flat[idx], real_dtype)

    def slice_load(self, array, start, size, dtype=None):
        a = np.asarray(array)
        return self.load(a[tuple(slice(s, s + n) for s, n in zip(start, size))], dtype)

    def stridedslice_load(self, array, start, end, step, dtype=None):
        a = np.asarray(array)
        return self.load(a[tuple(slice(s, e, p) for s, e, p in zip(start, end, step))], dtype)

    def view_store_expect(self, x, stride, e, eps=None):
        e = np.asarray(e)
        out = np.zeros(e.size, x.a.dtype)
        idx = np.zeros(x.a.shape, np.int64)
        for d, (n, st) in enumerate(zip(x.a.shape, stride)):
            ext = [1] * x.a.ndim
            ext[d] = n
            idx = idx + (np.arange(n, dtype=np.int64) * int(st)).reshape(ext)
        out[idx.reshape(-1)] = x.a.reshape(-1)
        v = OVal(out.reshape(e.shape), x.t)
        self.stores.append(v)
        return v

    # Gathers, one-hot, padded stores, element_any (include/dvm.h:284,297-307,344,482-496 of the reference; expected
    # values of tests/ut/test_gather_load.py, test_onehot.py:22-38, test_pad.py, test_element_any.py):
    #  * gather_mode 0: out[i0..in] = data[i0 .. index[i0..in] (at `axis`) .. in] (NumPy take_along_axis), gather_mode 1:
    #    the index's dims replace `axis` (NumPy take); a negative index counts from the end of the axis. What an index
    #    outside [-n, n) reads is not defined by the reference; the product clips it into the axis and so does this.
    #  * one_hot: a dim of extent depth at position axis, on_value where the position equals the index, off_value
    #    elsewhere (an index outside [0, depth) matches no position).
    #  * pad_store: the value written into the first columns of a zero-filled buffer whose innermost rows are pad
    #    elements longer.
    #  * element_any: the maximum over every element, as one fp32 value of shape [1].
    def global_access(self, array, dtype=None):
        return self.load(array, "int32" if dtype is None else dtype)

    def gather_load(self, data, index, axis=0, dtype=None, gather_mode=0):
        src = self.load(data, dtype)
        n = src.a.shape[axis]
        ix = index.a.astype(np.int64)
        ix = np.clip(np.where(ix < 0, ix + n, ix), 0, n - 1)
        ax = axis % src.a.ndim
        if gather_mode == 1:
            out = np.empty(src.a.shape[:ax] + ix.shape + src.a.shape[ax + 1:], src.a.dtype)
            for pos in np.ndindex(*ix.shape):
                out[(slice(None),) * ax + pos] = src.a[(slice(None),) * ax + (int(ix[pos]),)]
        else:
            out = np.empty(ix.shape, src.a.dtype)
            for pos in np.ndindex(*ix.shape):
                at = list(pos)
                at[ax] = int(ix[pos])
                out[pos] = src.a[tuple(at)]
        return OVal(out, src.t)

    def one_hot(self, indices, depth, axis, on_value, off_value, dtype):
        t = _tid(dtype)
        ix = indices.a
        ax = axis if axis >= 0 else ix.ndim + axis + 1
        shape = ix.shape[:ax] + (int(depth),) + ix.shape[ax:]
        np_t = np.int32 if t == I32 else np.float32
        out = np.full(shape, self._enc(off_value, t), np_t)
        on = self._enc(on_value, t)
        for pos in np.ndindex(*ix.shape):
            i = int(ix[pos])
            if 0 <= i < depth:
                out[pos[:ax] + (i,) + pos[ax:]] = on
        return OVal(out, t)

    def pad_store(self, x, pad):
        out = np.zeros(x.a.shape[:-1] + (x.a.shape[-1] + int(pad),), x.a.dtype)
        out[..., :x.a.shape[-1]] = x.a
        v = OVal(out, x.t)
        self.stores.append(v)
        return v

    def element_any(self, x):
        assert x.t == F32, "element_any needs fp32 input"
        return OVal(reduce_f32(1, x.a, list(range(x.a.ndim)), False).reshape(1), F32)

    def clear_store_memory(self, store):
        pass

    def full(self, scalar, shape, dtype):
        t = _tid(dtype)
        if t == BOOL:
            return self.cast(self.full(scalar, shape, F16), BOOL)
        return OVal(np.full(tuple(shape), self._enc(scalar, t), np.int32 if t == I32 else np.float32), t)

    @staticmethod
    def _enc(s, t):
        """A Python scalar converted to the tensor's type like EncodeScalar (src/dvm.cc:202-223)."""
        if t == I32:
            return np.int32(int(s))
        if t == BOOL:
            return np.float32(1.0 if s else 0.0)
        v = np.float32(s)
        if t == F16:
            return f16_bits_to_f32(f32_to_f16_bits(np.array([v])))[0]
        if t == BF16:
            return bf16_bits_to_f32(f32_to_bf16_bits(np.array([v])))[0]
        return v

    # -- casts --
    def _cast_step(self, x, t):
        s = x.t
        a = x.a
        if s == BOOL:
            return OVal(a.astype(np.float32), t)  # bool -> fp16: 1.0 / 0.0
        if t == BOOL:
            return OVal(a != 0, BOOL)
        if t == I32:
            out = np.empty(a.shape, np.int32)
            src = _c(a, np.float32)
            _lib().ora_f_to_i32(_p(src), _p(out), ctypes.c_size_t(src.size))
            return OVal(out, I32)
        if s == I32:
            src = _c(a, np.int32)
            out = np.empty(a.shape, np.float32)
            _lib().ora_i32_to_f(t, _p(src), _p(out), ctypes.c_size_t(src.size))
            return OVal(out, t)
        return OVal(round_to(t, a), t)

    def _noloss(self, x, t):
        while x.t != t:
            x = self._cast_step(x, _ROUTE[x.t][t])
        return x

    def cast(self, x, dtype):
        t = _tid(dtype)
        if x.t == t:
            return x
        if t == BOOL and not x.bool_result:
            return self.not_equal(x, 0)
        while x.t != t:
            x = self._cast_step(x, _ROUTE[x.t][t])
        return x

    # -- unary --
    def _unary(self, op, x):
        if x.t == BOOL:
            return self._noloss(self._unary(op, self._noloss(x, F16)), BOOL)
        if x.t == BF16:
            return self.cast(self._unary(op, self.cast(x, F32)), BF16)
        if x.t == F16 and ROUND <= op <= TRUNC:
            return self.cast(self._unary(op, self.cast(x, F32)), F16)
        if op == LNOT:
            return self.sub(1, x)
        if op == RECIP:
            return self.div(1, x)
        if x.t == I32:
            assert op == ABS
            src = _c(x.a, np.int32)
            out = np.empty(src.shape, np.int32)
            _lib().ora_abs_i32(_p(src), _p(out), ctypes.c_size_t(src.size))
            return OVal(out, I32)
        return OVal(unary_f(op, x.t, x.a), x.t)

    # -- binary --
    def _tensor_binary(self, op, l, r):
        if l.t == BOOL:
            return self._noloss(self._tensor_binary(op, self._noloss(l, F16), self._noloss(r, F16)), BOOL)
        if l.t == BF16 and op in (POW, DIV):
            return self.cast(self._tensor_binary(op, self.cast(l, F32), self.cast(r, F32)), BF16)
        if l.t == F16 and op == POW:
            return self.cast(self._tensor_binary(op, self.cast(l, F32), self.cast(r, F32)), F16)
        if op <= LE:
            c = OVal(compare(op, l.a, r.a, l.t == I32), l.t, bool_result=True)
            out = self._noloss(c, BOOL)
            out.bool_result = True
            return out
        if l.t == I32:
            return OVal(binary_i32(op, l.a, r.a), I32)
        return OVal(binary_f(op, l.t, l.a, r.a), l.t, bool_result=op in (LAND, LOR))

    def _scalar_binary(self, op, s, x, rhs_val):
        """x (op) s when rhs_val else s (op) x; None when the reference has no scalar form."""
        if op in (ADD, MUL, MAXIMUM, MINIMUM):
            sv = OVal(np.array(self._enc(s, x.t)), x.t)
            return self._plain(op, x, sv)
        if op == DIV:
            if x.t == BF16:
                return self.cast(self._scalar_binary(op, s, self.cast(x, F32), rhs_val), BF16)
            sv = OVal(np.array(self._enc(s, x.t)), x.t)
            return self._plain(op, x, sv) if rhs_val else self._plain(op, sv, x)
        if op <= LE:
            sv = OVal(np.array(self._enc(s, x.t)), x.t)
            l, r = (x, sv) if rhs_val else (sv, x)
            c = OVal(compare(op, l.a, r.a, x.t == I32), x.t, bool_result=True)
            out = self._noloss(c, BOOL)
            out.bool_result = True
            return out
        if op == POW:
            if rhs_val:
                if isinstance(s, (int, np.integer)) or float(s) == math.floor(float(s)):
                    return self._pow_int(x, int(s), isinstance(s, (int, np.integer)))
                return None
            if float(s) > 0:
                if x.t != F32:
                    return self.cast(self._scalar_binary(POW, float(s), self.cast(x, F32), False), x.t)
                lg = np.float32(math.log(np.float32(s)))
                return self._unary(EXP, self._scalar_binary(MUL, lg, x, True))
            return None
        if op == SUB:
            if rhs_val:
                return self._scalar_binary(ADD, -s, x, True)
            m1 = -1 if isinstance(s, (int, np.integer)) else -1.0
            return self._scalar_binary(ADD, s, self._scalar_binary(MUL, m1, x, True), True)
        return None

    def _plain(self, op, l, r):
        if l.t == I32:
            return OVal(binary_i32(op, l.a, r.a), I32)
        return OVal(binary_f(op, l.t, l.a, r.a), l.t, bool_result=op in (LAND, LOR))

    def _pow_int(self, x, n, int_scalar):
        it = abs(n)
        if it == 0:
            return self.full(1 if int_scalar else 1.0, x.shape(), x.t)
        res = None
        if it == 1:
            res = x
        else:
            while it:
                if it & 1:
                    res = x if res is None else self._tensor_binary(MUL, res, x)
                if it != 1:
                    x = self._tensor_binary(MUL, x, x)
                it >>= 1
        if n < 0:
            res = self._unary(RECIP, res)
        return res

    def _binary(self, op, l, r):
        if isinstance(l, OVal) and isinstance(r, OVal):
            return self._tensor_binary(op, l, r)
        x, s, rhs_val = (l, r, True) if isinstance(l, OVal) else (r, l, False)
        if x.t == BOOL:
            xf = self._noloss(x, F16)
            out = self._binary(op, xf, s) if rhs_val else self._binary(op, s, xf)
            return self._noloss(out, BOOL)
        out = self._scalar_binary(op, s, x, rhs_val)
        if out is None:
            b = self.full(s, x.shape(), x.t)
            out = self._tensor_binary(op, x, b) if rhs_val else self._tensor_binary(op, b, x)
        return out

    def select(self, cond, lhs, rhs):
        c = self._noloss(cond, lhs.t) if cond.t != lhs.t else cond
        ca, la, ra = np.broadcast_arrays(c.a, lhs.a, rhs.a)
        return OVal(np.where(ca != 0, la, ra), lhs.t)

    # -- shape ops --
    def broadcast(self, x, shape):
        shape = list(shape)
        for i, d in enumerate(shape):
            if d == -1:
                shape[i] = x.a.shape[x.a.ndim + i - len(shape)]
        return OVal(np.broadcast_to(x.a, shape).copy(), x.t, x.bool_result)

    def reshape(self, x, shape):
        return OVal(x.a.reshape(tuple(shape)), x.t, x.bool_result)

    # views of values (include/dvm.h:434,443,453,479 of the reference): NumPy's transpose and basic slicing
    def permute(self, x, dims):
        return OVal(np.ascontiguousarray(np.transpose(x.a, tuple(dims))), x.t, x.bool_result)

    def slice(self, x, start, size):
        idx = tuple(slice(s + (n if s < 0 else 0), s + (n if s < 0 else 0) + k) for s, k, n in zip(start, size, x.a.shape))
        return OVal(np.ascontiguousarray(x.a[idx]), x.t, x.bool_result)

    def slice_dim(self, x, dim, begin, end):
        idx = [slice(None)] * x.a.ndim
        idx[dim] = slice(begin, end)
        return OVal(np.ascontiguousarray(x.a[tuple(idx)]), x.t, x.bool_result)

    def concat(self, inputs, dim):
        return OVal(np.concatenate([x.a for x in inputs], axis=dim), inputs[0].t, inputs[0].bool_result)

    def split(self, x, dim, split_size, split_num):
        return tuple(self.slice_dim(x, dim, j * split_size, (j + 1) * split_size) for j in range(split_num))

    def copy(self, x):
        return OVal(x.a.copy(), x.t, x.bool_result)

    # -- reduce --
    def _reduce(self, kind, x, dims, keepdims):
        if isinstance(dims, int):
            dims = (dims,)
        if kind == 0:
            assert x.t == F32, "sum needs fp32 input"
        if x.t == I32:
            # max / min of integers: order-independent and exact; fp32 would not hold values above 2^24
            fn = np.max if kind == 1 else np.min
            return OVal(fn(x.a, axis=tuple(d % x.a.ndim for d in dims), keepdims=keepdims).astype(np.int32), x.t)
        return OVal(reduce_f32(kind, x.a, list(dims), keepdims), x.t)

    def sum(self, x, dims, keepdims=False):
        return self._reduce(0, x, dims, keepdims)

    def max(self, x, dims, keepdims=False):
        return self._reduce(1, x, dims, keepdims)

    def min(self, x, dims, keepdims=False):
        return self._reduce(2, x, dims, keepdims)

    def matmul(self, lhs, rhs, trans_a, trans_b, bias=None):
        return OVal(matmul(lhs.a, rhs.a, bias.a if bias is not None else None, trans_a, trans_b, lhs.t), lhs.t)

    def grouped_matmul(self, lhs, rhs, trans_a, trans_b, bias, group_list, group_type, group_list_type=0):
        """One product per group (include/dvm.h:510-522, src/ops_m.cc:721-762 of the reference; expected values of
        tests/ut/test_gmm.py:25-76): the list holds the groups' upper bounds (group_list_type 0) or sizes (1).
        group_type 0: rows [lo, hi) of lhs times matrix g of rhs (+ row g of the bias) are rows [lo, hi) of the
        result; rows past the last bound are left at zero here (the product does not write them). group_type 2:
        columns [lo, hi) of lhs times rows [lo, hi) of rhs (+ row g of the bias) are matrix g of the result. Every
        product is the matmul of this module: fp32 accumulation, bias added in fp32, one rounding."""
        a = lhs.a.T if trans_a else lhs.a
        b = np.swapaxes(rhs.a, -1, -2) if trans_b else rhs.a
        gl = np.asarray(group_list.a, np.int64)
        if group_list_type == 1:
            gl = np.cumsum(gl)
        m, k = a.shape
        lim = m if group_type == 0 else k
        gl = np.clip(gl, 0, lim)
        n = b.shape[-1]
        out = np.zeros((m, n) if group_type == 0 else (len(gl), m, n), np.float32)
        lo = 0
        for g, hi in enumerate(gl):
            hi = max(int(hi), lo)
            bg = bias.a[g] if bias is not None else None
            if group_type == 0:
                if hi > lo:
                    out[lo:hi] = matmul(np.ascontiguousarray(a[lo:hi]), np.ascontiguousarray(b[g]), bg, False, False, lhs.t)
            elif hi > lo:
                out[g] = matmul(np.ascontiguousarray(a[:, lo:hi]), np.ascontiguousarray(b[lo:hi]), bg, False, False, lhs.t)
            elif bg is not None:
                out[g] = np.broadcast_to(round_to(lhs.t, bg.astype(np.float32)), (m, n))
            lo = hi
        return OVal(out, lhs.t)

    # -- outputs --
    def store(self, x, dtype=None):
        if dtype is not None:
            x = self.cast(x, dtype)
        self.stores.append(x)
        return x

    def output(self, x):
        """The stored tensor as the numpy array a caller of the product would read back."""
        if x.t == F16:
            return x.a.astype(np.float16)
        return x.a


def _add_named_ops():
    un = ["sqrt", "abs", "log", "exp", "reciprocal", "isfinite", "logical_not", "round", "floor", "ceil", "trunc"]
    bi = ["equal", "not_equal", "greater", "greater_equal", "less", "less_equal", "add", "sub", "mul", "div", "pow",
          "maximum", "minimum", "logical_and", "logical_or"]
    for i, n in enumerate(un):
        setattr(OracleKernel, n, (lambda idx: lambda self, x: self._unary(idx, x))(i))
    for i, n in enumerate(bi):
        setattr(OracleKernel, n, (lambda idx: lambda self, l, r: self._binary(idx, l, r))(i))


_add_named_ops()
