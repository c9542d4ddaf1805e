"""Seeded random graphs for the parity tests: each generator returns a function that builds the same graph on the
HIP path (dvm_amd.tester.Tester) and on the CPU oracle (oracle.oracle.OracleKernel). Graphs are planned on the
oracle, whose shapes are known while the graph is built, and recorded as a tape that both builders replay.

pointwise_reduce_graph  fp32 arithmetic over fp32/fp16/bf16 inputs with broadcasts, reduces, reshapes, several outputs
typed_graph             values kept in their own types (fp32/fp16/bf16/int32/bool): compares, logic, selects, casts
matmul_graph            one matmul (transposes, batches, shared operands) with a computed operand and an epilogue chain
dynamic_case            one graph and three sets of input shapes for a kernel object built with -1 extents
view_graph              permute / slice / split / concat / copy chains mixed with pointwise operators and reduces
index_graph             one_hot / gather_load (both modes, computed indices) / pad_store / element_any around pointwise
                        operators, reduces, permutes and slices"""
import numpy as np

from dvm_amd.tester import Tester
from oracle.oracle import OracleKernel, BOOL, F16, BF16, F32, I32


def close_enough(out, ref, exact):
    """Bit-exact for integer and bool outputs; for floating point 2e-4, where up to 1% of the elements may differ
    by one step of a 16-bit format (exp and sums differ in the last fp32 bit between the device and NumPy, and a
    cast to fp16/bf16 after them can round to the neighbouring value)."""
    a, b = np.asarray(out).astype(np.float64), np.asarray(ref).astype(np.float64)
    if a.shape != b.shape:
        return False
    if exact:
        return np.array_equal(a, b)
    with np.errstate(all="ignore"):
        d = np.abs(a - b)
        bad = ~(d <= 2e-4 + 2e-4 * np.abs(b)) & ~(np.isnan(a) & np.isnan(b)) & ~(a == b)
        return not bad.any() or (bad.mean() < 0.01 and np.nanmax(np.where(bad, d / (np.abs(b) + 1e-3), 0)) < 1e-2)


# further operators of the generator below (more=True): reduces to the minimum, over two axes and without keepdims,
# logarithm, reciprocal square root, minimum, numbers on either side
MORE_OPS = ["min", "sum2", "sumnk", "log", "abs", "rsqrt", "minimum", "square", "recip", "maxnk", "mulc", "subc"]


def pointwise_reduce_graph(case, big=False, more=False):
    rng = np.random.default_rng(case)
    rank = int(rng.integers(1, 4))
    big = int(big)
    shape = [int(rng.choice([1, 2, 3, 7, 16, 33, 64] + ([130, 500] if big else []))) for _ in range(rank)]
    shape[-1] = int(rng.choice([1, 5, 8, 24, 64, 100, 257, 1024] + ([4096, 10000, 40000] if big else [])))
    while int(np.prod(shape)) > (1 << 21): shape[int(np.argmax(shape[:-1]))] = 1 if rank > 1 and max(shape[:-1]) > 1 else shape.__setitem__(-1, 1024) or 1
    n_in = int(rng.integers(1, 4))
    ins = []
    for i in range(n_in):
        sh = list(shape)
        for d in range(rank):
            if rng.random() < 0.25: sh[d] = 1
        dt = str(rng.choice(["float32", "float32", "float16", "bfloat16"]))
        arr = rng.uniform(0.25, 2.0, sh).astype(np.float32)
        ins.append((arr, dt))
    prog = [(str(rng.choice(["add", "mul", "sub", "div", "exp", "sqrt", "cast16", "castbf", "cast32", "sum", "max", "bcast", "select", "neg", "maximum", "reshape", "addc"] + (MORE_OPS if more else []))), int(rng.integers(0, 1 << 30))) for _ in range(int(rng.integers(2, 9 + 6 * big)))]
    n_out = int(rng.integers(1, 3 + big))
    # plan the graph on the oracle (its shapes are known at once) and record it as a tape both builders replay
    tape = []
    def plan():
        k = OracleKernel()
        vals = [k.cast(k.load(arr if dt == "float32" else (arr.astype(np.float16) if dt == "float16" else arr), None if dt != "bfloat16" else "bfloat16"), "float32") for arr, dt in ins]
        for name, seed in prog:
            r = np.random.default_rng(seed)
            xi, yi = int(r.integers(0, len(vals))), int(r.integers(0, len(vals)))
            x, y = vals[xi], vals[yi]
            xs, ys = tuple(x.shape()), tuple(y.shape())
            try:
                np.broadcast_shapes(xs, ys); compat = True
            except ValueError:
                compat = False
            step = None
            if name in ("add", "mul", "sub", "div", "maximum") and compat: step = (name, xi, yi, None)
            elif name in ("exp", "sqrt", "cast16", "castbf", "cast32", "neg", "log", "abs", "rsqrt", "square", "recip"): step = (name, xi, None, None)
            elif name == "minimum" and compat: step = (name, xi, yi, None)
            elif name in ("mulc", "subc"): step = (name, xi, None, float(r.random()) + 0.5)
            elif name in ("min", "sumnk", "maxnk") and len(xs) > 0: step = (name, xi, None, int(r.integers(0, len(xs))))
            elif name == "sum2" and len(xs) > 1: step = (name, xi, None, tuple(sorted({int(r.integers(0, len(xs))), int(r.integers(0, len(xs)))})))
            elif name == "addc": step = (name, xi, None, float(r.random()))
            elif name in ("sum", "max") and len(xs) > 0: step = (name, xi, None, int(r.integers(0, len(xs))))
            elif name == "bcast" and len(xs) > 0:
                try:
                    step = (name, xi, None, list(shape)) if np.broadcast_shapes(xs, tuple(shape)) == tuple(shape) and len(xs) == len(shape) else None
                except ValueError:
                    pass
            elif name == "select" and compat: step = (name, xi, yi, None)
            elif name == "reshape" and len(xs) >= 2: step = (name, xi, None, [int(np.prod(xs))])
            if step is None: continue
            if compat and step[2] is not None and int(np.prod(np.broadcast_shapes(xs, ys))) > (1 << 22): continue
            tape.append(step)
            vals.append(apply(k, vals, step))
    def apply(k, vals, step):
        name, xi, yi, prm = step
        x = vals[xi]; y = vals[yi] if yi is not None else None
        f32 = lambda v: k.cast(v, "float32")
        if name == "div": return k.div(x, k.add(k.abs(y), 0.5))
        if name in ("add", "mul", "sub", "maximum"): return getattr(k, name)(x, y)
        if name == "exp": return k.exp(k.mul(x, 0.125))
        if name == "sqrt": return k.sqrt(k.abs(x))
        if name == "cast16": return f32(k.cast(x, "float16"))
        if name == "castbf": return f32(k.cast(x, "bfloat16"))
        if name == "cast32": return f32(x)
        if name in ("sum", "max"): return getattr(k, name)(x, (prm,), True)
        if name == "min": return k.min(x, (prm,), True)
        if name == "sumnk": return k.sum(x, (prm,), False)
        if name == "maxnk": return k.max(x, (prm,), False)
        if name == "sum2": return k.sum(x, prm, True)
        if name == "log": return k.log(k.add(k.abs(x), 0.25))
        if name == "abs": return k.abs(x)
        if name == "rsqrt": return k.div(1.0, k.sqrt(k.add(k.abs(x), 0.25)))
        if name == "square": return k.mul(x, x)
        if name == "recip": return k.reciprocal(k.add(k.abs(x), 0.5))
        if name == "minimum": return k.minimum(x, y)
        if name == "mulc": return k.mul(x, prm)
        if name == "subc": return k.sub(prm, x)
        if name == "bcast": return k.broadcast(x, prm)
        if name == "select": return k.select(k.greater(x, y), x, y)
        if name == "neg": return k.mul(x, -1.0)
        if name == "addc": return k.add(x, prm)
        if name == "reshape": return k.reshape(x, prm)
    plan()
    def build(k):
        vals = []
        for arr, dt in ins:
            if dt == "float32": v = k.load(arr)
            elif dt == "float16": v = k.load(arr.astype(np.float16))
            else: v = k.load(arr, "bfloat16")
            vals.append(k.cast(v, "float32"))
        for step in tape:
            vals.append(apply(k, vals, step))
        return [k.store(v) for v in vals[-n_out:]]
    return build


UN_F = ["sqrt_abs", "abs", "log1", "exp8", "recip", "round", "floor", "ceil", "trunc", "isfinite"]
BIN = ["add", "sub", "mul", "maximum", "minimum", "div"]
CMP = ["equal", "not_equal", "greater", "greater_equal", "less", "less_equal"]

def typed_graph(case):
    rng = np.random.default_rng(case)
    rank = int(rng.integers(1, 4))
    shape = [int(rng.choice([1, 2, 3, 7, 16, 33, 64, 130])) for _ in range(rank)]
    shape[-1] = int(rng.choice([1, 5, 8, 24, 64, 100, 257, 1024, 4096]))
    ins = []
    for i in range(int(rng.integers(1, 4))):
        sh = list(shape)
        for d in range(rank):
            if rng.random() < 0.25: sh[d] = 1
        dt = str(rng.choice(["float32", "float16", "bfloat16", "int32", "int32", "bool"]))
        if dt == "int32": arr = rng.integers(-50, 50, sh).astype(np.int32)
        elif dt == "bool": arr = rng.random(sh) < 0.5
        elif dt == "float16": arr = rng.uniform(-2, 2, sh).astype(np.float16)
        else: arr = rng.uniform(-2, 2, sh).astype(np.float32)
        ins.append((arr, dt))
    n_steps = int(rng.integers(2, 12)); n_out = int(rng.integers(1, 4))
    tape = []
    def apply(k, vals, step):
        name, xi, yi, prm = step
        x = vals[xi]; y = vals[yi] if yi is not None else None
        if name == "sqrt_abs": return k.sqrt(k.abs(x))
        if name == "log1": return k.log(k.add(k.abs(x), 1.0))
        if name == "exp8": return k.exp(k.mul(x, 0.125))
        if name == "recip": return k.reciprocal(k.add(k.abs(x), 0.5))
        if name == "div": return k.div(x, k.add(k.abs(y), 0.5))
        if name in ("abs", "round", "floor", "ceil", "trunc", "isfinite", "logical_not"): return getattr(k, name)(x)
        if name in BIN or name in CMP or name in ("logical_and", "logical_or"): return getattr(k, name)(x, y)
        if name == "select": return k.select(vals[prm], x, y)
        if name == "cast": return k.cast(x, prm)
        if name in ("sum", "max", "min"): return getattr(k, name)(x, (prm[0],), prm[1])
        if name == "bcast": return k.broadcast(x, prm)
        if name == "addc": return k.add(x, prm)
        if name == "reshape": return k.reshape(x, prm)
        raise KeyError(name)
    def load(k, arr, dt):
        return k.load(arr, "bfloat16") if dt == "bfloat16" else k.load(arr)
    def plan():
        k = OracleKernel()
        vals = [load(k, a, d) for a, d in ins]
        for _ in range(n_steps):
            xi = int(rng.integers(0, len(vals))); x = vals[xi]; xs = tuple(x.shape())
            same = [j for j, v in enumerate(vals) if v.t == x.t]
            yi = int(rng.choice(same)); ys = tuple(vals[yi].shape())
            try:
                bs = np.broadcast_shapes(xs, ys); compat = int(np.prod(bs)) <= (1 << 21)
            except ValueError:
                compat = False
            fl = x.t in (F16, BF16, F32)
            kinds = ["cast", "cast", "bcast", "reshape"]
            if fl: kinds += ["un", "un", "bin", "bin", "cmp", "red", "addc", "select"]
            elif x.t == I32: kinds += ["abs", "bin", "bin", "cmp", "cmp", "addc", "select"]
            else: kinds += ["logic", "logic", "lnot", "select"]
            kind = str(rng.choice(kinds)); step = None
            if kind == "un": step = (str(rng.choice(UN_F)), xi, None, None)
            elif kind == "abs": step = ("abs", xi, None, None)
            elif kind == "bin" and compat:
                nm = str(rng.choice(BIN if fl else BIN[:5])); step = (nm, xi, yi, None)
            elif kind == "cmp" and compat: step = (str(rng.choice(CMP)), xi, yi, None)
            elif kind == "logic" and compat: step = (str(rng.choice(["logical_and", "logical_or"])), xi, yi, None)
            elif kind == "lnot": step = ("logical_not", xi, None, None)
            elif kind == "addc": step = ("addc", xi, None, float(np.round(rng.uniform(-2, 2), 2)) if fl else int(rng.integers(-5, 5)))
            elif kind == "select" and compat:
                bools = [j for j, v in enumerate(vals) if v.t == BOOL]
                if bools:
                    ci = int(rng.choice(bools))
                    try:
                        if int(np.prod(np.broadcast_shapes(bs, tuple(vals[ci].shape())))) <= (1 << 21): step = ("select", xi, yi, ci)
                    except ValueError:
                        pass
            elif kind == "cast": step = ("cast", xi, None, str(rng.choice(["float32", "float16", "bfloat16", "int32", "bool"])))
            elif kind == "red" and len(xs) > 0:
                nm = str(rng.choice(["sum", "max", "min"]))
                if nm != "sum" or x.t == F32: step = (nm, xi, None, (int(rng.integers(0, len(xs))), bool(rng.random() < 0.5)))
            elif kind == "bcast" and len(xs) == len(shape) and all(a in (1, b) for a, b in zip(xs, shape)): step = ("bcast", xi, None, list(shape))
            elif kind == "reshape" and len(xs) >= 2: step = ("reshape", xi, None, [int(np.prod(xs))])
            if step is None: continue
            try:
                v = apply(k, vals, step)
            except Exception:
                continue
            tape.append(step); vals.append(v)
    plan()
    def build(k):
        vals = [load(k, a, d) for a, d in ins]
        for step in tape: vals.append(apply(k, vals, step))
        return [k.store(v) for v in vals[-n_out:]]
    build.tape = tape; build.ins = ins
    return build


def matmul_graph(case):
    rng = np.random.default_rng(case)
    M = int(rng.choice([1, 7, 64, 130, 256, 300, 513])); N = int(rng.choice([1, 8, 64, 130, 256, 300, 520]))
    K = int(rng.choice([8, 64, 100, 256, 1000])); ta, tb = bool(rng.random() < 0.5), bool(rng.random() < 0.5)
    dt = str(rng.choice(["float16", "bfloat16"]))
    batch = [[], [], [2], [3, 1], [2, 2]][int(rng.integers(0, 5))]
    ba = list(batch); bb = list(batch)
    if batch and rng.random() < 0.4: bb = []          # rhs shared by the batch
    elif batch and rng.random() < 0.3: ba = [1] * len(batch)
    sa = ba + ([K, M] if ta else [M, K]); sb = bb + ([N, K] if tb else [K, N])
    mk = lambda sh: (rng.normal(0, 0.3, sh).astype(np.float32))
    a, b = mk(sa), mk(sb)
    steps = []
    for _ in range(int(rng.integers(0, 6))):
        kind = str(rng.choice(["rowvec", "colvec", "full", "un", "addc", "cast16", "select", "mulc"]))
        if kind == "rowvec": steps.append((kind, mk([N]), str(rng.choice(["add", "mul", "sub"]))))
        elif kind == "colvec": steps.append((kind, mk([M, 1]), str(rng.choice(["add", "mul", "maximum"]))))
        elif kind == "full": steps.append((kind, mk(list(np.broadcast_shapes(ba or [1], bb or [1])) + [M, N]) if batch and rng.random() < 0.5 else mk([M, N]), str(rng.choice(["add", "mul", "sub", "minimum"]))))
        elif kind == "un": steps.append((kind, None, str(rng.choice(["abs", "exp8", "sqrt_abs", "neg", "sigmoid"]))))
        elif kind == "addc": steps.append((kind, float(np.round(rng.uniform(-1, 1), 2)), None))
        elif kind == "mulc": steps.append((kind, float(np.round(rng.uniform(-2, 2), 2)), None))
        else: steps.append((kind, None, None))
    f32_epi = bool(rng.random() < 0.6); both = bool(rng.random() < 0.3); pro = bool(rng.random() < 0.2)
    def ld(k, arr):
        return k.load(arr, "bfloat16") if dt == "bfloat16" else k.load(arr.astype(np.float16))
    def build(k):
        A, B = ld(k, a), ld(k, b)
        if pro: A = k.cast(k.mul(k.cast(A, "float32"), 0.5), dt)   # a computed operand: its own launch before the product
        c = k.matmul(A, B, ta, tb)
        outs = [c] if both or not steps else []
        x = k.cast(c, "float32") if f32_epi else c
        for kind, arr, op in steps:
            if kind in ("rowvec", "colvec", "full"):
                o = ld(k, arr)
                if f32_epi: o = k.cast(o, "float32")
                x = getattr(k, op)(x, o)
            elif kind == "un":
                if op == "abs": x = k.abs(x)
                elif op == "exp8": x = k.exp(k.mul(x, 0.125))
                elif op == "sqrt_abs": x = k.sqrt(k.abs(x))
                elif op == "neg": x = k.mul(x, -1.0)
                else: x = k.div(x, k.add(k.exp(k.mul(x, -1.0)), 1.0))
            elif kind == "addc": x = k.add(x, arr)
            elif kind == "mulc": x = k.mul(x, arr)
            elif kind == "cast16": x = k.cast(k.cast(x, dt), "float32") if f32_epi else x
            elif kind == "select": x = k.select(k.greater(x, 0.0), x, k.mul(x, 0.1))
        if steps or not outs: outs.append(k.cast(x, dt) if f32_epi and rng_out_cast else x)
        return [k.store(o) for o in outs]
    rng_out_cast = bool(rng.random() < 0.7)
    build.desc = (M, N, K, ta, tb, dt, sa, sb, [(s[0], s[2]) for s in steps], f32_epi, both, pro)
    return build


DYN_OPS = ["add", "mul", "sub", "div", "exp", "sqrt", "cast16", "castbf", "sum", "max", "min", "select", "neg", "maximum", "addc"]

def dyn_apply(k, vals, step):
    name, xi, yi, prm = step
    x = vals[xi]; y = vals[yi] if yi is not None else None
    f32 = lambda v: k.cast(v, "float32")
    if name == "div": return k.div(x, k.add(k.abs(y), 0.5))
    if name in ("add", "mul", "sub", "maximum"): return getattr(k, name)(x, y)
    if name == "exp": return k.exp(k.mul(x, 0.125))
    if name == "sqrt": return k.sqrt(k.abs(x))
    if name == "cast16": return f32(k.cast(x, "float16"))
    if name == "castbf": return f32(k.cast(x, "bfloat16"))
    if name in ("sum", "max", "min"): return getattr(k, name)(x, (prm[0],), prm[1])
    if name == "select": return k.select(k.greater(x, y), x, y)
    if name == "neg": return k.mul(x, -1.0)
    if name == "addc": return k.add(x, prm)

def dynamic_case(case):
    rng = np.random.default_rng(case)
    rank = int(rng.integers(1, 4)); n_in = int(rng.integers(1, 4))
    ones = [[bool(rng.random() < 0.25) for _ in range(rank)] for _ in range(n_in)]
    dts = [str(rng.choice(["float32", "float32", "float16"])) for _ in range(n_in)]
    insts = []
    for _ in range(3):
        shape = [int(rng.choice([1, 2, 3, 7, 16, 33, 64, 130])) for _ in range(rank)]
        shape[-1] = int(rng.choice([1, 5, 8, 24, 64, 100, 257, 1024, 4096]))
        insts.append([rng.uniform(0.25, 2.0, [1 if o else s for o, s in zip(on, shape)]).astype(dt) for on, dt in zip(ones, dts)])
    ks = [OracleKernel() for _ in insts]
    vals = [[k.cast(k.load(a), "float32") for a in ins] for k, ins in zip(ks, insts)]
    tape = []
    for _ in range(int(rng.integers(2, 11))):
        name = str(rng.choice(DYN_OPS)); n = len(vals[0])
        xi, yi = int(rng.integers(0, n)), int(rng.integers(0, n))
        rk = len(vals[0][xi].shape())
        if name in ("sum", "max", "min"):
            if rk == 0: continue
            step = (name, xi, None, (int(rng.integers(0, rk)), bool(rng.random() < 0.6)))
        elif name in ("add", "mul", "sub", "div", "select", "maximum"): step = (name, xi, yi, None)
        elif name == "addc": step = (name, xi, None, float(np.round(rng.uniform(0, 1), 2)))
        else: step = (name, xi, None, None)
        try:
            new = [dyn_apply(k, v, step) for k, v in zip(ks, vals)]
            if len({len(v.shape()) for v in new}) != 1: continue
        except Exception:
            continue
        tape.append(step)
        for v, nv in zip(vals, new): v.append(nv)
    n_out = int(rng.integers(1, 4))
    refs = [[k.output(k.store(x)) for x in v[-n_out:]] for k, v in zip(ks, vals)]
    return insts, dts, tape, n_out, refs


def view_graph(case):
    rng = np.random.default_rng(case)
    with_op_first = bool(rng.integers(0, 2))
    rank = int(rng.integers(2, 5))
    shape = [int(rng.choice([1, 2, 3, 5, 8, 16, 33, 64, 100])) for _ in range(rank)]
    shape[-1] = int(rng.choice([8, 24, 64, 100, 128, 257]))
    a = rng.standard_normal(shape).astype(np.float32)
    b = rng.standard_normal(shape).astype(np.float32)
    ops = []
    n_ops = int(rng.integers(1, 6))
    for _ in range(n_ops):
        ops.append((str(rng.choice(["permute", "slice", "slice_dim", "split", "concat", "add", "mul", "sum", "reshape_copy", "view_load"])), int(rng.integers(0, 1 << 30))))
    def build(k):
        x = k.add(k.load(a), 0.5) if with_op_first else k.load(a)
        cur_shape = list(shape)
        stores = []
        for name, seed in ops:
            r = np.random.default_rng(seed)
            rk = len(cur_shape)
            if name == "permute":
                perm = list(r.permutation(rk))
                x = k.permute(x, [int(p) for p in perm]); cur_shape = [cur_shape[p] for p in perm]
            elif name == "slice":
                start = [int(r.integers(0, n)) for n in cur_shape]
                size = [int(r.integers(1, n - s + 1)) for n, s in zip(cur_shape, start)]
                x = k.slice(x, start, size); cur_shape = size
            elif name == "slice_dim":
                d = int(r.integers(0, rk)); n = cur_shape[d]
                b0 = int(r.integers(0, n)); e0 = int(r.integers(b0 + 1, n + 1))
                x = k.slice_dim(x, d, b0, e0); cur_shape[d] = e0 - b0
            elif name == "split":
                d = int(r.integers(0, rk)); n = cur_shape[d]
                if n < 2: continue
                cs = int(r.integers(1, n)); num = (n + cs - 1) // cs
                parts = k.split(x, d, cs, num)
                pick = int(r.integers(0, num))
                if num > 1 and r.random() < 0.5:
                    other = parts[(pick + 1) % num]
                    stores.append(k.store(k.mul(other, 2.0)))
                x = parts[pick]; cur_shape[d] = min(cs, n - pick * cs)
            elif name == "concat":
                d = int(r.integers(0, rk))
                y = k.mul(x, -1.0)
                x = k.concat([x, y, x], d); cur_shape[d] *= 3
            elif name == "add":
                x = k.add(x, float(r.random()))
            elif name == "mul":
                x = k.mul(x, x)
            elif name == "sum":
                d = int(r.integers(0, rk))
                x = k.sum(x, (d,), True); cur_shape[d] = 1
            elif name == "reshape_copy":
                tot = int(np.prod(cur_shape))
                x = k.reshape(k.copy(x), [tot]); cur_shape = [tot]
                if tot % 4 == 0:
                    x = k.reshape(x, [tot // 4, 4]); cur_shape = [tot // 4, 4]
            elif name == "view_load":
                if list(cur_shape) == list(shape):
                    x = k.add(x, k.load(b))
        stores.append(k.store(x))
        return stores
    return build



def index_graph(case):
    rng = np.random.default_rng(case)
    rank = int(rng.integers(1, 4))
    shape = [int(rng.choice([1, 2, 3, 5, 8, 17, 40])) for _ in range(rank)]
    shape[-1] = int(rng.choice([1, 3, 8, 24, 64, 100, 257]))
    dt = str(rng.choice(["float32", "float32", "float16", "bfloat16", "int32"]))
    kind = str(rng.choice(["onehot", "take", "along"]))
    axis = int(rng.integers(0, rank + (1 if kind == "onehot" else 0)))
    if rng.random() < 0.3:
        axis -= rank + (1 if kind == "onehot" else 0)
    depth = int(rng.choice([1, 2, 7, 16, 100, 300]))
    ix_shape = [int(rng.choice([1, 2, 4, 9, 33])) for _ in range(int(rng.integers(1, 3)))]
    src = rng.integers(-50, 50, shape).astype(np.int32) if dt == "int32" else rng.uniform(-2, 2, shape).astype(np.float32)
    if dt == "float16": src = src.astype(np.float16)
    if kind == "onehot":
        ix = rng.integers(-2, depth + 2, shape).astype(np.int32)
    elif kind == "take":
        n = shape[axis]
        ix = rng.integers(-n - 3, n + 3, ix_shape).astype(np.int32)
    else:
        n = shape[axis]
        sh = list(shape)
        sh[axis] = int(rng.choice([1, 2, 5, 19]))
        ix = rng.integers(-n, n, sh).astype(np.int32)
    computed_ix = bool(rng.integers(0, 2))
    tail = [(str(rng.choice(["add", "mul", "sum", "max", "permute", "slice_dim", "any", "pad", "neg"])), int(rng.integers(0, 1 << 30)))
            for _ in range(int(rng.integers(0, 4)))]

    def head(k):
        i = k.load(ix)
        if computed_ix:
            i = k.sub(k.add(i, 3), 3)
        if kind == "onehot":
            if dt == "int32":
                return k.one_hot(i, depth, axis, 3, -1, dt)
            x = k.one_hot(i, depth, axis, 1.5, -0.25, dt)
            return x if dt == "float32" else k.cast(x, "float32")
        x = k.gather_load(src, i, axis=axis, dtype=dt, gather_mode=1 if kind == "take" else 0)
        return x if dt in ("float32", "int32") else k.cast(x, "float32")

    is_int = dt == "int32"

    def step(k, x, stores, op):
        name = op[0]
        if name == "add":
            return k.add(x, 2 if is_int else 0.5)
        if name == "mul":
            return k.mul(x, x)
        if name == "neg":
            return k.mul(x, -1 if is_int else -1.0)
        if name in ("sum", "max"):
            return (k.sum if name == "sum" else k.max)(x, (op[1],), op[2])
        if name == "permute":
            return k.permute(x, list(op[1]))
        if name == "slice_dim":
            return k.slice_dim(x, op[1], op[2], op[3])
        if name == "any":
            stores.append(k.store(k.element_any(k.abs(x))))
        elif name == "pad":
            stores.append(k.pad_store(k.add(x, 1 if is_int else 1.0), op[1]))
        return x

    # the graph is planned on the oracle, whose shapes are known while it is built, and recorded as a tape
    tape = []
    with np.errstate(all="ignore"):
        ko = OracleKernel()
        x = head(ko)
        for name, seed in tail:
            r = np.random.default_rng(seed)
            shp = list(x.shape())
            rk = len(shp)
            op = None
            if name in ("add", "mul", "neg"):
                op = (name,)
            elif name in ("sum", "max") and rk > 0 and not (name == "sum" and is_int):
                op = (name, int(r.integers(0, rk)), bool(r.integers(0, 2)))
            elif name == "permute" and rk > 1:
                op = (name, [int(p) for p in r.permutation(rk)])
            elif name == "slice_dim" and rk > 0:
                d = int(r.integers(0, rk)); n = shp[d]
                if n >= 1:
                    b0 = int(r.integers(0, n)); e0 = int(r.integers(b0 + 1, n + 1))
                    op = (name, d, b0, e0)
            elif name == "any" and not is_int and rk > 0:
                op = (name,)
            elif name == "pad" and rk > 0:
                op = (name, int(r.integers(0, 9)))
            if op is not None:
                tape.append(op)
                x = step(ko, x, [], op)

    def build(k):
        x = head(k)
        stores = []
        for op in tape:
            x = step(k, x, stores, op)
        stores.append(k.store(x))
        return stores
    return build


def compile_in_das_mode(seeds):
    """The host compiler alone on `seeds` cases of every generator, in disassembly mode (no GPU): what `make
    asan-check` runs against the sanitizer build. A compile error with one of the documented messages is a valid
    outcome; anything else, or a sanitizer report, ends the run."""
    from dvm_amd.tester import Tester
    from oracle.oracle import OracleKernel
    done = refused = 0
    for case in range(seeds):
        for gen, ker in ((lambda c: pointwise_reduce_graph(c, True), ""), (typed_graph, ""), (matmul_graph, "mix"), (view_graph, ""), (index_graph, "")):
            build = gen(case)
            if gen is not matmul_graph:
                try:  # (the plan of a graph is made on the oracle; a case it rejects is no case)
                    build(OracleKernel())
                except Exception:  # noqa: BLE001
                    continue
            t = Tester(ker, run_mode="das")
            try:
                build(t)
                t.codegen()
                t.das()
                done += 1
            except RuntimeError as e:
                if not any(s in str(e) for s in ("needs a Copy", "not supported", "too many")):
                    raise RuntimeError("case %d: %s" % (case, e)) from e
                refused += 1
    return done, refused


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("--das-seeds", type=int, default=200)
    n_done, n_refused = compile_in_das_mode(ap.parse_args().das_seeds)
    print("compiled %d random graphs in disassembly mode, %d refused with a documented error" % (n_done, n_refused))
