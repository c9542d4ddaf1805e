"""GPU parity at and beyond the ends of the float ranges: every unary, binary, scalar, cast, reduce and compare
operator on zeros of both signs, infinities, NaN, the largest and smallest floats, denormals, rounding ties and the
int32 limits, in three float types, alone and inside a sweep behind a reduce; and matmul epilogues on products that
overflow, underflow and cancel. The HIP path against the oracle (whose functors are the reference's,
src/vm_gpu.cu:198-329): same NaNs and infinities in the same places, finite values within the type's tolerance."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from oracle.oracle import OracleKernel

pytestmark = pytest.mark.gpu

FMAX = np.finfo(np.float32).max
TINY = np.finfo(np.float32).tiny
VALUES = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, np.inf, -np.inf, np.nan, FMAX, -FMAX, 3e38, -3e38, 2.4e38,
                   -2.4e38, TINY, -TINY, TINY / 4, 1e-45, -1e-45, 65504.0, -65504.0, 65520.0, 70000.0, 1e-8, 6e-8, 88.0,
                   -88.0, 89.0, -104.0, -150.0, 1e10, -1e10, 2147483647.0, 2147483648.0, -2147483648.0, -2147483904.0, 4e9,
                   0.49999997, 1.5, 2.5, -1.5, -2.5, 3.5, 8388607.5, 16777216.0, 1e-20, 1e20, 3.0, -3.0, 0.1, 255.0, 256.0,
                   -7.0], np.float32)
FLOATS = ["float32", "float16", "bfloat16"]
UNARY = ["sqrt", "abs", "log", "exp", "reciprocal", "round", "floor", "ceil", "trunc", "isfinite", "neg", "rsqrt", "tanh",
         "sigmoid"]
BINARY = ["add", "sub", "mul", "div", "maximum", "minimum", "pow"]


def unary(k, name, x):
    if name == "neg":
        return k.mul(x, -1.0)
    if name == "rsqrt":
        return k.div(1.0, k.sqrt(x))
    if name == "tanh":
        e = k.exp(k.mul(x, 2.0))
        return k.div(k.sub(e, 1.0), k.add(e, 1.0))
    if name == "sigmoid":
        return k.div(1.0, k.add(k.exp(k.mul(x, -1.0)), 1.0))
    return getattr(k, name)(x)


def load_as(k, arr, dt):
    if dt == "float32":
        return k.load(arr)
    if dt == "float16":
        with np.errstate(over="ignore"):
            return k.load(arr.astype(np.float16))
    if dt == "bfloat16":
        return k.load(arr, "bfloat16")
    with np.errstate(all="ignore"):
        return k.load(np.clip(np.nan_to_num(arr, nan=0, posinf=2e9, neginf=-2e9), -2.1e9, 2.1e9).astype(np.int32))


def agree(tag, build, ker="vector", tol=2e-3):
    t, o = Tester(ker), OracleKernel()
    st, so = t.store(build(t)), o.store(build(o))
    t.run()
    out, ref = np.asarray(t.output(st)), np.asarray(o.output(so))
    if out.dtype == np.uint16:  # bf16 comes back as its bits from the device, as values from the oracle
        out = Tester.convert_from_bf16(out)
    if ref.dtype == np.uint16:
        ref = Tester.convert_from_bf16(ref)
    assert out.shape == ref.shape, tag
    if out.dtype.kind in "ib":
        bad = out != ref
    else:
        a, b = out.astype(np.float64), ref.astype(np.float64)
        with np.errstate(all="ignore"):
            bad = ~((np.isnan(a) & np.isnan(b)) | (a == b) | (np.abs(a - b) <= 1e-5 + tol * np.abs(b)))
    if bad.any():
        i = np.flatnonzero(bad.ravel())[:6]
        raise AssertionError("%s: %d elements differ, e.g. at %s: hip %s, oracle %s\n%s"
                             % (tag, int(bad.sum()), i.tolist(), out.ravel()[i], ref.ravel()[i], t.das()))


@pytest.mark.parametrize("dt", FLOATS)
def test_unary_operators_alone_and_inside_a_sweep(dt):
    x = np.tile(VALUES, 4)
    rows = np.tile(VALUES, (8, 20))  # rows of 1120 behind a row maximum: the sweep build
    ones = np.ones_like(rows)
    for name in UNARY:
        agree("%s %s" % (name, dt), lambda k: unary(k, name, load_as(k, x, dt)))

        def in_sweep(k):
            top = k.max(k.load(ones), (1,), True)
            return unary(k, name, k.mul(k.cast(load_as(k, rows, dt), "float32"), top))
        agree("%s %s in a sweep" % (name, dt), in_sweep)


@pytest.mark.parametrize("dt", FLOATS)
def test_binary_operators_on_every_pair(dt):
    a, b = np.repeat(VALUES, len(VALUES)), np.tile(VALUES, len(VALUES))
    for name in BINARY:
        agree("%s %s" % (name, dt), lambda k: getattr(k, name)(load_as(k, a, dt), load_as(k, b, dt)))


@pytest.mark.parametrize("dt", FLOATS)
def test_operators_with_a_number_on_either_side(dt):
    x = np.tile(VALUES, 4)
    for name in BINARY:
        for s in [0.0, -0.0, 2.0, -1.0, 0.5, np.inf, 3.0]:
            if name == "pow" and (dt != "float32" or s == np.inf):
                continue
            agree("%s %s x, %r" % (name, dt, s), lambda k: getattr(k, name)(load_as(k, x, dt), float(s)))
            agree("%s %s %r, x" % (name, dt, s), lambda k: getattr(k, name)(float(s), load_as(k, x, dt)))


@pytest.mark.parametrize("src,dst", [("float32", "float16"), ("float32", "bfloat16"), ("float32", "int32"), ("float16", "float32"),
                                     ("float16", "int32"), ("bfloat16", "float32"), ("float32", "bool"), ("int32", "float32"),
                                     ("float16", "bfloat16")])
def test_casts(src, dst):
    x = np.tile(VALUES, 4)
    agree("%s -> %s" % (src, dst), lambda k: k.cast(load_as(k, x, src), dst))


@pytest.mark.parametrize("dt", ["float32", "float16"])
def test_reduces_over_rows_and_columns_that_hold_them(dt):
    rows = np.stack([np.roll(VALUES, i)[:40] for i in range(len(VALUES))]).astype(np.float32)
    for name in ["sum", "max", "min"]:
        if name == "sum" and dt != "float32":
            continue
        for axis in (1, 0):
            agree("%s %s axis %d" % (name, dt, axis), lambda k: getattr(k, name)(load_as(k, rows, dt), (axis,), True))


def test_compares_on_every_pair():
    a, b = np.repeat(VALUES, len(VALUES)), np.tile(VALUES, len(VALUES))
    for name in ["equal", "not_equal", "greater", "greater_equal", "less", "less_equal"]:
        agree(name, lambda k: getattr(k, name)(k.load(a), k.load(b)))


# ---- matmul epilogues: the products are the values of B (A has a single one per row) ----

PRODUCTS = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -2.0, 65504.0, -65504.0, 6e-8, -6e-8, 6.1e-5, 88.0, -88.0, 89.0, -104.0, 11.0,
                     -11.0, 12.0, 16.0, -17.0, 100.0, -100.0, 30000.0, -30000.0, 3.0, 7.0, 0.1, -0.1, 255.0, 1e-3, -1e-3,
                     20.0], np.float32)
EPILOGUES = {
    "plain": lambda k, z: z,
    "exp": lambda k, z: k.exp(z),
    "exp of the negative": lambda k, z: k.exp(k.mul(z, -1.0)),
    "reciprocal": lambda k, z: k.div(1.0, z),
    "silu": lambda k, z: k.div(z, k.add(k.exp(k.mul(z, -1.0)), 1.0)),
    "sigmoid": lambda k, z: k.div(1.0, k.add(k.exp(k.mul(z, -1.0)), 1.0)),
    "log": lambda k, z: k.log(z),
    "sqrt": lambda k, z: k.sqrt(z),
    "inf - inf": lambda k, z: k.sub(k.mul(z, 1e35), k.mul(z, 1e35)),
    "relu": lambda k, z: k.maximum(z, 0.0),
    "min with 1": lambda k, z: k.minimum(z, 1.0),
    "round of abs": lambda k, z: k.round(k.abs(z)),
    "tanh": lambda k, z: (lambda e: k.div(k.sub(e, 1.0), k.add(e, 1.0)))(k.exp(k.mul(z, 2.0))),
    "x / x": lambda k, z: k.div(z, z),
    "select": lambda k, z: k.select(k.greater(z, 0.0), k.exp(z), k.mul(z, 2.0)),
}


@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
@pytest.mark.parametrize("mnk", [(128, 128, 64), (300, 200, 96), (64, 520, 32)])
def test_matmul_epilogues_on_products_at_the_ends_of_the_range(dt, mnk):
    m, n, kk = mnk
    a = np.zeros([m, kk], np.float32)
    a[np.arange(m), np.arange(m) % kk] = 1.0
    b = np.stack([np.roll(PRODUCTS, r)[np.arange(n) % len(PRODUCTS)] for r in range(kk)])
    bias_row = np.linspace(-3, 3, n).astype(np.float32)
    for out_dt in (dt, "float32"):
        for name, f in EPILOGUES.items():
            for bias in (False, True):
                def build(k):
                    x, y = load_as(k, a, dt), load_as(k, b, dt)
                    mm = k.matmul(x, y, False, False, k.load(bias_row)) if bias else k.matmul(x, y, False, False)
                    return k.cast(f(k, k.cast(mm, "float32")), out_dt)
                agree("%s %s -> %s, %s, bias %s" % (dt, mnk, out_dt, name, bias), build, ker="mix",
                      tol=1e-2 if out_dt != "float32" else 2e-3)
