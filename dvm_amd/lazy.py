"""Eager fusion without graphs for PyTorch: `with dvm_amd.lazy_fusion():` makes the supported operators on GPU tensors
append to a pending DVM graph instead of launching one kernel each; whatever needs values ends the segment, and the
pending operators run as fused launches.

The role of the reference's "Eager lazy fusion" (docs/pytorch.md, section 4: the operator sequence of an eager
program is captured as it is issued, fusable runs become DVM kernels, everything else falls back operator by
operator). There the capture sits in the framework's operator plugin and is switched on by an environment variable;
here it is a `torch.utils._python_dispatch.TorchDispatchMode`, switched on by a `with` block:

  * a captured operator returns its result tensor at once (allocated, not yet written) and records a node;
  * an operator outside the table below, an operator on types or layouts the table does not take, an in-place or
    `out=` form, a copy to the host, `item()`: the pending segment is flushed first when the operator touches memory
    the segment reads or writes, then the operator runs as usual (the fallback is automatic, per operator);
  * `flush()`, leaving the block, or 48 pending operators flush as well. `torch.cuda.synchronize()` does not pass
    through the dispatcher: call `flush()` (or leave the block) before waiting for results by other means;
  * a result nobody holds any more when the segment runs (the temporaries of an expression) is never stored: it lives
    in registers of the fused kernel.

Compiled segments are kept by signature (operators, shapes, strides, types, constants): a loop that issues the same
sequence again binds new addresses and launches. Launches go to torch's current stream; workspace comes from torch's
caching allocator.
"""
import math
import weakref

import torch
from torch.utils._python_dispatch import TorchDispatchMode

from ._core import DataType, PyKernel

aten = torch.ops.aten

_DT = {torch.float32: DataType.float32, torch.float16: DataType.float16, torch.bfloat16: DataType.bfloat16,
       torch.bool: DataType.bool, torch.int32: DataType.int32}
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)
_MAX_PENDING = 48


class _Node:
    __slots__ = ("op", "args", "shape", "dtype", "out", "const")

    def __init__(self, op, args, shape, dtype, out, const=()):
        self.op, self.args, self.shape, self.dtype, self.const = op, args, tuple(shape), dtype, tuple(const)
        self.out = weakref.ref(out)


def _number(v):
    """A Python number, or the number a zero-dim CPU tensor wraps (how `x + 1.0` may arrive); else None."""
    if isinstance(v, bool):
        return None
    if isinstance(v, (int, float)):
        return v
    if isinstance(v, torch.Tensor) and v.dim() == 0 and not v.is_cuda and v.dtype in (torch.float32, torch.float64, torch.int64, torch.int32):
        return v.item()
    return None


def _broadcast(*shapes):
    """NumPy's rule, on tuples (torch.broadcast_shapes costs more than everything else a captured operator does)."""
    first = shapes[0]
    if all(s == first for s in shapes[1:]):
        return tuple(first)
    rank = max(len(s) for s in shapes)
    out = [1] * rank
    for s in shapes:
        for i, n in enumerate(s):
            j = rank - len(s) + i
            if n != 1:
                if out[j] != 1 and out[j] != n:
                    return None
                out[j] = n
    return tuple(out)


class LazyFusion(TorchDispatchMode):
    def __init__(self, ktype="eager"):
        super().__init__()
        self._ktype = ktype
        self._nodes = []       # pending operators, in issue order
        self._inputs = []      # tensors the segment reads (kept alive until it has run)
        self._input_index = {}  # id(tensor) -> position in _inputs
        self._node_of = {}     # id(result tensor) -> position in _nodes
        self._storages = set()  # storages the segment reads or writes
        self._cache = {}
        self._alive = []
        self.stats = {"captured": 0, "fallbacks": 0, "flushes": 0, "launches": 0, "compiled": 0, "stored": 0}

    # ---- capture ----
    def _operand(self, t, matrix=False):
        """('n', i): result of pending node i; ('i', j): input tensor j; None: not a tensor this mode takes.
        `matrix`: a matmul operand, which may also be a transposed view (its rows contiguous instead of its columns)."""
        if not isinstance(t, torch.Tensor) or type(t) not in (torch.Tensor, torch.nn.Parameter) or not t.is_cuda or t.dtype not in _DT or t.is_sparse:
            return None
        i = self._node_of.get(id(t))
        if i is not None and self._nodes[i].out() is t:
            return ("n", i)
        if t.numel() == 0 or t.dim() > 8 or any(s < 0 for s in t.stride()):
            return None
        if t.dim() > 0 and t.stride(-1) != 1 and t.shape[-1] != 1 and not t.is_contiguous():
            if not (matrix and t.dim() >= 2 and t.stride(-2) == 1):
                return None  # (a view without a contiguous innermost axis: left to torch)
        j = self._input_index.get(id(t))
        if j is None or self._inputs[j] is not t:
            j = len(self._inputs)
            self._inputs.append(t)
            self._input_index[id(t)] = j
            self._storages.add(t.untyped_storage().data_ptr())
        return ("i", j)

    def _emit(self, op, args, shape, dtype, device, const=()):
        out = torch.empty(tuple(shape), dtype=dtype, device=device)
        self._node_of[id(out)] = len(self._nodes)
        self._nodes.append(_Node(op, args, shape, dtype, out, const))
        self._storages.add(out.untyped_storage().data_ptr())
        self.stats["captured"] += 1
        if len(self._nodes) >= _MAX_PENDING:
            self.flush()
        return out

    def _unary(self, op, x, floats_only=True, const=()):
        a = self._operand(x)
        if a is None or (floats_only and x.dtype not in _FLOATS):
            return NotImplemented
        return self._emit(op, (a,), x.shape, x.dtype, x.device, const)

    def _binary(self, op, x, y, out_dtype=None, alpha=1):
        if alpha != 1:
            return NotImplemented
        xs, ys = _number(x), _number(y)
        if xs is not None and ys is not None:
            return NotImplemented
        t = y if xs is not None else x
        if not isinstance(t, torch.Tensor) or t.dtype not in _FLOATS + (torch.int32,):
            return NotImplemented
        if isinstance(xs, float) or isinstance(ys, float):
            if t.dtype == torch.int32:
                return NotImplemented  # (type promotion: left to torch)
        if t.dtype == torch.int32 and op in ("div", "pow"):
            return NotImplemented
        if xs is None and ys is None:
            if x.dtype != y.dtype or x.device != y.device:
                return NotImplemented
            a, b = self._operand(x), self._operand(y)
            if a is None or b is None:
                return NotImplemented
            shape = _broadcast(x.shape, y.shape)
            if shape is None:
                return NotImplemented
            return self._emit(op, (a, b), shape, out_dtype or x.dtype, x.device)
        a = self._operand(t)
        if a is None:
            return NotImplemented
        if xs is not None:  # scalar on the left
            return self._emit(op, (a,), t.shape, out_dtype or t.dtype, t.device, ("l", xs))
        return self._emit(op, (a,), t.shape, out_dtype or t.dtype, t.device, ("r", ys))

    def _where(self, c, x, y):
        if not all(isinstance(v, torch.Tensor) for v in (c, x, y)) or c.dtype != torch.bool or x.dtype != y.dtype or x.dtype not in _FLOATS:
            return NotImplemented
        ops = [self._operand(v) for v in (c, x, y)]
        if any(o is None for o in ops):
            return NotImplemented
        shape = _broadcast(c.shape, x.shape, y.shape)
        if shape is None:
            return NotImplemented
        return self._emit("where", tuple(ops), shape, x.dtype, x.device)

    def _cast(self, x, kwargs):
        extra = {k: v for k, v in kwargs.items() if v is not None and k not in ("dtype", "non_blocking", "copy")}
        dtype = kwargs.get("dtype")
        if extra or dtype is None or dtype not in _DT or dtype == x.dtype or x.dtype not in _DT:
            return NotImplemented
        a = self._operand(x)
        if a is None:
            return NotImplemented
        return self._emit("cast", (a,), x.shape, dtype, x.device)

    def _sum(self, x, dim=None, keepdim=False, dtype=None):
        if x.dtype not in _FLOATS or (dtype is not None and dtype != x.dtype) or x.dim() == 0:
            return NotImplemented
        a = self._operand(x)
        if a is None:
            return NotImplemented
        dims = list(range(x.dim())) if dim is None or len(dim) == 0 else sorted({d % x.dim() for d in dim})
        shape = [1 if i in dims else n for i, n in enumerate(x.shape)] if keepdim else [n for i, n in enumerate(x.shape) if i not in dims]
        return self._emit("sum", (a,), shape, x.dtype, x.device, (tuple(dims), bool(keepdim)))

    def _matmul(self, x, y, bias=None, beta=1, alpha=1):
        if beta != 1 or alpha != 1 or x.dtype != y.dtype or x.dtype not in (torch.float16, torch.bfloat16):
            return NotImplemented
        if x.dim() != y.dim() or x.dim() not in (2, 3) or (x.dim() == 3 and x.shape[0] != y.shape[0]):
            return NotImplemented
        if bias is not None and (bias.dtype != x.dtype or bias.dim() != 1 or bias.shape[0] != y.shape[-1] or x.dim() != 2):
            return NotImplemented
        ops = [self._operand(x, True), self._operand(y, True)] + ([self._operand(bias)] if bias is not None else [])
        if any(o is None for o in ops):
            return NotImplemented
        return self._emit("matmul", tuple(ops), tuple(x.shape[:-1]) + (y.shape[-1],), x.dtype, x.device)

    def __torch_dispatch__(self, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        handler = _TABLE.get(func)
        if handler is not None:
            try:
                out = handler(self, *args, **kwargs)
            except TypeError:
                out = NotImplemented
            if out is not NotImplemented:
                return out
        self.stats["fallbacks"] += 1
        if self._nodes and self._touches_segment(args, kwargs):
            self.flush()
        return func(*args, **kwargs)

    def _touches_segment(self, args, kwargs):
        def walk(v):
            if isinstance(v, torch.Tensor):
                try:
                    return v.is_cuda and v.untyped_storage().data_ptr() in self._storages
                except (RuntimeError, NotImplementedError):
                    return True
            if isinstance(v, (list, tuple)):
                return any(walk(e) for e in v)
            return False
        return walk(args) or walk(tuple(kwargs.values()))

    def __exit__(self, *exc):
        try:
            if exc[0] is None:
                self.flush()
            else:
                self._drop()
        finally:
            super().__exit__(*exc)

    def _drop(self):
        self._nodes, self._inputs, self._input_index, self._node_of, self._storages = [], [], {}, {}, set()

    # ---- running a segment ----
    def flush(self):
        """Compiles (or finds) the kernel of the pending operators and launches it on torch's current stream."""
        if not self._nodes:
            return
        nodes, inputs = self._nodes, self._inputs
        self._drop()
        outs = [n.out() for n in nodes]
        stored = [i for i, o in enumerate(outs) if o is not None]
        if not stored:
            return
        device = inputs[0].device if inputs else next(o for o in outs if o is not None).device
        sig = (tuple((n.op, n.args, n.shape, n.dtype, n.const) for n in nodes),
               tuple((tuple(t.shape), tuple(t.stride()) if not t.is_contiguous() else None, t.dtype) for t in inputs), tuple(stored), device.index)
        entry = self._cache.get(sig)
        if entry is None:
            entry = self._build(nodes, inputs, stored, device)
            self._cache[sig] = entry
            self.stats["compiled"] += 1
        k, loads, stores = entry
        with torch.utils._python_dispatch._disable_current_modes():
            for ld, t in zip(loads, inputs):
                shape = tuple(t.shape) if t.dim() > 0 else (1,)
                if t.is_contiguous():
                    k.bind_device(ld, t.data_ptr(), shape)
                else:
                    k.bind_device(ld, t.data_ptr(), shape, strides=tuple(t.stride()))
            for st, i in zip(stores, stored):
                k.bind_device(st, outs[i].data_ptr())
            scratch = []

            def workspace(nbytes):
                scratch.append(torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device))
                return scratch[-1].data_ptr()

            k.set_workspace_allocator(workspace)
            k.codegen()
            k.run(stream=torch.cuda.current_stream(device).cuda_stream, sync=False, on_given_stream=True)
        self._alive = [inputs, outs, scratch]  # until the next segment has been queued behind this one
        self.stats["flushes"] += 1
        self.stats["launches"] += k.num_launches()
        self.stats["stored"] += len(stored)

    def _build(self, nodes, inputs, stored, device):
        k = PyKernel(self._ktype, "dev", device.index or 0)
        loads = [k.load(list(t.shape) if t.dim() > 0 else [1], _DT[t.dtype]) for t in inputs]
        vals = []

        def val(ref):
            return loads[ref[1]] if ref[0] == "i" else vals[ref[1]]

        for n in nodes:
            a = [val(r) for r in n.args]
            vals.append(_BUILD[n.op](k, n, a))
        stores = []
        for i in stored:
            v = vals[i]
            if int(v.dtype()) != int(_DT[nodes[i].dtype]):
                v = k.cast(v, _DT[nodes[i].dtype])
            stores.append(k.store(v))
        return k, loads, stores


# ---- how a captured operator is written with the DVM builder ----

def _f32(k, x):
    return x if int(x.dtype()) == int(DataType.float32) else k.cast(x, DataType.float32)


def _back(k, n, x):
    return x if int(x.dtype()) == int(_DT[n.dtype]) else k.cast(x, _DT[n.dtype])


def _scalar_binary(name, widen=False):
    """widen: arithmetic of a 16-bit tensor with a number happens in fp32 with the number as it is and is rounded
    once, as torch's kernels do it (the DVM operator alone would first round the number to the tensor's type);
    compares take the number in the tensor's type on both sides."""
    def build(k, n, a):
        fn = getattr(k, name)
        if len(a) == 2:
            return fn(a[0], a[1])
        side, s = n.const
        x = a[0]
        narrow = widen and int(x.dtype()) in (int(DataType.float16), int(DataType.bfloat16))
        if narrow:
            x = k.cast(x, DataType.float32)
        out = fn(s, x) if side == "l" else fn(x, s)
        return k.cast(out, _DT[n.dtype]) if narrow else out
    return build


def _in_f32(body):
    """16-bit operands are widened, the result is rounded once: how torch's own kernels compute these."""
    def build(k, n, a):
        return _back(k, n, body(k, n, _f32(k, a[0])))
    return build


_BUILD = {
    "add": _scalar_binary("add", True), "sub": _scalar_binary("sub", True), "mul": _scalar_binary("mul", True),
    "div": _scalar_binary("div", True), "pow": _scalar_binary("pow", True),
    "maximum": _scalar_binary("maximum"), "minimum": _scalar_binary("minimum"),
    "eq": _scalar_binary("equal"), "ne": _scalar_binary("not_equal"), "gt": _scalar_binary("greater"),
    "ge": _scalar_binary("greater_equal"), "lt": _scalar_binary("less"), "le": _scalar_binary("less_equal"),
    "abs": lambda k, n, a: k.abs(a[0]),
    "neg": lambda k, n, a: k.mul(a[0], -1 if n.dtype == torch.int32 else -1.0),
    "sqrt": lambda k, n, a: k.sqrt(a[0]),
    "exp": lambda k, n, a: k.exp(a[0]),
    "log": lambda k, n, a: k.log(a[0]),
    "reciprocal": lambda k, n, a: k.reciprocal(a[0]),
    "rsqrt": _in_f32(lambda k, n, x: k.div(1.0, k.sqrt(x))),
    "relu": lambda k, n, a: k.maximum(a[0], 0.0),
    "leaky_relu": _in_f32(lambda k, n, x: k.select(k.greater(x, 0.0), x, k.mul(x, float(n.const[0])))),
    "sigmoid": _in_f32(lambda k, n, x: k.div(1.0, k.add(k.exp(k.mul(x, -1.0)), 1.0))),
    "silu": _in_f32(lambda k, n, x: k.div(x, k.add(k.exp(k.mul(x, -1.0)), 1.0))),
    # 1 - 2 / (exp(2x) + 1): finite at both ends (exp overflows to inf, 2 / inf is 0)
    "tanh": _in_f32(lambda k, n, x: k.sub(1.0, k.div(2.0, k.add(k.exp(k.mul(x, 2.0)), 1.0)))),
    # the tanh approximation: 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3)))
    "gelu_tanh": _in_f32(lambda k, n, x: k.mul(k.mul(x, 0.5), k.sub(2.0, k.div(2.0, k.add(k.exp(k.mul(k.mul(k.add(k.mul(k.mul(k.mul(x, x), x), 0.044715), x), math.sqrt(2.0 / math.pi)), 2.0)), 1.0))))),
    "where": lambda k, n, a: k.select(a[0], a[1], a[2]),
    "cast": lambda k, n, a: k.cast(a[0], _DT[n.dtype]),
    "sum": lambda k, n, a: _back(k, n, k.sum(_f32(k, a[0]), list(n.const[0]), n.const[1])),
    "matmul": lambda k, n, a: k.matmul(a[0], a[1], False, False, a[2] if len(a) > 2 else None),
}


def _bin(op, out_dtype=None):
    def handler(self, x, y, alpha=1):
        return self._binary(op, x, y, out_dtype, alpha)
    return handler


def _un(op, floats_only=True):
    return lambda self, x: self._unary(op, x, floats_only)


def _gelu(self, x, approximate="none"):
    return self._unary("gelu_tanh", x) if approximate == "tanh" else NotImplemented


def _leaky(self, x, negative_slope=0.01):
    return self._unary("leaky_relu", x, True, (float(negative_slope),))


def _pow(self, x, y):
    return self._binary("pow", x, y) if _number(y) is not None and isinstance(x, torch.Tensor) and x.dtype in _FLOATS else NotImplemented


_TABLE = {
    aten.add.Tensor: _bin("add"), aten.add.Scalar: _bin("add"), aten.sub.Tensor: _bin("sub"), aten.sub.Scalar: _bin("sub"),
    aten.mul.Tensor: _bin("mul"), aten.mul.Scalar: _bin("mul"), aten.div.Tensor: _bin("div"), aten.div.Scalar: _bin("div"),
    aten.rsub.Scalar: lambda self, x, other, alpha=1: self._binary("sub", other, x, None, alpha),
    aten.maximum.default: _bin("maximum"), aten.minimum.default: _bin("minimum"),
    aten.pow.Tensor_Scalar: _pow,
    aten.eq.Tensor: _bin("eq", torch.bool), aten.eq.Scalar: _bin("eq", torch.bool), aten.ne.Tensor: _bin("ne", torch.bool),
    aten.ne.Scalar: _bin("ne", torch.bool), aten.gt.Tensor: _bin("gt", torch.bool), aten.gt.Scalar: _bin("gt", torch.bool),
    aten.ge.Tensor: _bin("ge", torch.bool), aten.ge.Scalar: _bin("ge", torch.bool), aten.lt.Tensor: _bin("lt", torch.bool),
    aten.lt.Scalar: _bin("lt", torch.bool), aten.le.Tensor: _bin("le", torch.bool), aten.le.Scalar: _bin("le", torch.bool),
    aten.abs.default: _un("abs", False), aten.neg.default: _un("neg", False), aten.sqrt.default: _un("sqrt"),
    aten.exp.default: _un("exp"), aten.log.default: _un("log"), aten.reciprocal.default: _un("reciprocal"),
    aten.rsqrt.default: _un("rsqrt"), aten.relu.default: _un("relu"), aten.sigmoid.default: _un("sigmoid"),
    aten.silu.default: _un("silu"), aten.tanh.default: _un("tanh"), aten.gelu.default: _gelu, aten.leaky_relu.default: _leaky,
    aten.where.self: lambda self, c, x, y: self._where(c, x, y),
    aten._to_copy.default: lambda self, x, **kw: self._cast(x, kw),
    aten.sum.dim_IntList: lambda self, x, dim=None, keepdim=False, dtype=None: self._sum(x, dim, keepdim, dtype),
    aten.sum.default: lambda self, x, dtype=None: NotImplemented,  # (a zero-dim result: left to torch)
    aten.mm.default: lambda self, x, y: self._matmul(x, y),
    aten.bmm.default: lambda self, x, y: self._matmul(x, y),
    aten.addmm.default: lambda self, bias, x, y, beta=1, alpha=1: self._matmul(x, y, bias, beta, alpha),
}


def lazy_fusion(ktype="eager"):
    """`with lazy_fusion() as lf: ...` - see the module text. `lf.flush()` runs what is pending; `lf.stats` counts
    captured operators, fallbacks, segments, launches and stored results."""
    return LazyFusion(ktype)
