"""GPU parity: element-wise, scalar, logical, cast, compare and select graphs.

Each case restates a gpu-marked case of the reference's tests/ut (cited per test): same shapes,
same input distributions, NumPy golden and tolerance (fp32 1e-5, fp16 1e-3, bf16 1e-2, integers
and bools exact); the graph additionally runs on the CPU oracle and both results must agree."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_unary(dt):  # tests/ut/test_elemwise.py:24-35
    x = np.full([32, 1024], 0.5, dt)
    run_parity(lambda k, a: [k.sqrt(a), k.abs(a), k.log(a), k.exp(a), k.reciprocal(a)], [x],
               golden=[np.sqrt(x), np.abs(x), np.log(x), np.exp(x), np.reciprocal(x)])


def test_exp_at_the_ends_of_the_range():
    # the lowest float is what a masked softmax fills in (tests/ut/test_pass_insert_removepad.py:99): its product
    # with log2(e) overflows although the value is finite; results below the smallest normal number may come out as 0
    fmax = np.finfo(np.float32).max
    vals = np.array([-fmax, fmax, -3e38, -2.4e38, -2.3e38, 2.4e38, -np.inf, np.inf, np.nan, -104.0, -103.0, -88.0,
                     -87.3, 0.0, -0.0, 88.0, 88.7, 89.0, 1e-30, -1e-30], np.float32)
    x = np.tile(vals, 64).reshape(64, -1)
    with np.errstate(over="ignore"):
        gold = np.exp(x)

    masked = np.tile(np.array([-fmax, -3e38, -2.4e38, -104.0, -88.0, 0.0, 1.0, 5.0], np.float32), 512).reshape(4, -1)
    with np.errstate(over="ignore"):
        soft = np.exp(masked - masked.max(axis=1, keepdims=True))

    def g(k, a, m):  # alone, after an arithmetic operator, and in the sweep behind a row maximum
        return [k.exp(a), k.exp(k.mul(a, 1.0)), k.exp(k.sub(m, k.max(m, (1,), True)))]
    run_parity(g, [x, masked], golden=[gold, gold, soft], golden_eps=1e-5)


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_binary(dt):  # tests/ut/test_elemwise.py:38-54
    x, y = np.full([32, 1024], 0.5, dt), np.full([32, 1024], 0.4, dt)

    def g(k, a, b):
        a, b = k.copy(a), k.copy(b)
        return [k.copy(k.add(a, b)), k.sub(a, b), k.div(a, b), k.mul(a, b), k.maximum(a, b), k.minimum(a, b)]
    run_parity(g, [x, y], golden=[x + y, x - y, x / y, x * y, np.maximum(x, y), np.minimum(x, y)])


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_binary_random_bit_exact_fp16(dt):
    rng = np.random.default_rng(11)
    x, y = rng.normal(0, 1, [64, 1000]).astype(dt), rng.normal(0, 1, [64, 1000]).astype(dt)
    outs = run_parity(lambda k, a, b: [k.add(a, b), k.sub(a, b), k.mul(a, b), k.div(a, b)], [x, y], eps=0,
                      golden=[x + y, x - y, x * y, x / y], golden_eps=0)
    assert outs[0].dtype == dt


@pytest.mark.parametrize("shape", [(1024, 32), (1312, 131), (16, 11), (128, 7), (128, 777)])
@pytest.mark.parametrize("dt", [np.bool_, np.float16, np.float32])
def test_logical(shape, dt):  # tests/ut/test_elemwise.py:57-109
    rng = np.random.default_rng(shape[1])
    x, y = rng.choice([True, False], shape).astype(dt), rng.choice([True, False], shape).astype(dt)
    outs = run_parity(lambda k, a, b: [k.logical_and(a, b), k.logical_or(a, b), k.logical_not(a)], [x, y])
    assert np.array_equal(outs[0].astype(bool), np.logical_and(x, y))
    assert np.array_equal(outs[1].astype(bool), np.logical_or(x, y))
    assert np.array_equal(outs[2].astype(bool), np.logical_not(x))


def test_logical_not_int32():
    x = np.random.default_rng(1).integers(0, 2, [128, 777]).astype(np.int32)
    outs = run_parity(lambda k, a: k.logical_not(a), [x])
    assert np.array_equal(outs[0], 1 - x)


def test_logical_on_compare_results_of_mixed_types():  # tests/ut/test_elemwise.py:76-94
    rng = np.random.default_rng(2)
    xi, yi = rng.integers(-1024, 1024, [128, 777]).astype(np.int32), rng.integers(-1024, 1024, [128, 777]).astype(np.int32)
    xf, yf = rng.normal(0, 1, [128, 777]).astype(np.float32), rng.normal(0, 1, [128, 777]).astype(np.float32)
    run_parity(lambda k, a, b, c, d: [k.logical_and(k.greater(a, b), k.less(c, d)), k.logical_or(k.greater(a, b), k.less(c, d))],
               [xi, yi, xf, yf], golden=[np.logical_and(xi > yi, xf < yf), np.logical_or(xi > yi, xf < yf)])


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_tensor_scalar(dt):  # tests/ut/test_elemwise.py:112-140
    rng = np.random.default_rng(3)
    x = rng.normal(0.05, 1, [32, 1024]).astype(dt)
    s = 0.1
    sd = dt(s)
    run_parity(lambda k, a: [k.add(a, s), k.mul(a, s), k.div(a, s), k.maximum(a, s), k.minimum(a, s), k.div(s, a), k.sub(s, a), k.sub(a, s)],
               [x], golden=[x + sd, x * sd, x / sd, np.maximum(x, sd), np.minimum(x, sd), sd / x, sd - x, x - sd])


@pytest.mark.parametrize("n", [1024, 24, 66666])
@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_isfinite(n, dt):  # tests/ut/test_elemwise.py:143-158
    rng = np.random.default_rng(n)
    x = rng.normal(0, 1, n).astype(dt)
    x[:: 7] = np.inf
    x[3:: 11] = -np.inf
    x[5:: 13] = np.nan
    rng.shuffle(x)
    outs = run_parity(lambda k, a: k.isfinite(a), [x], eps=0)
    assert np.array_equal(outs[0] != 0, np.isfinite(x))


def test_long_1d_and_single_element():  # tests/ut/test_elemwise.py:161-185
    x = np.full([32 * 64 * 257], 0.5, np.float32)
    run_parity(lambda k, a: k.add(a, 0.1), [x], golden=x + np.float32(0.1))
    a, b = np.full([1], 0.4, np.float32), np.full([1], 0.2, np.float32)
    run_parity(lambda k, p, q: k.sub(p, q), [a, b], golden=a - b)


def test_full_div():  # tests/ut/test_elemwise.py:205-216
    rng = np.random.default_rng(4)
    x = rng.uniform(0, 1, [2, 3, 4, 5]).astype(np.float16) + np.float16(0.1)
    run_parity(lambda k, a: k.div(k.full(2.0, [2, 3, 4, 5], "float16"), a), [x], golden=np.float16(2.0) / x)
    y = rng.uniform(0.1, 1, [1, 1, 4, 5]).astype(np.float32)
    run_parity(lambda k, a: k.div(k.full(2.0, [1, 1, 4, 5], "float32"), a), [y], golden=np.float32(2.0) / y)


def test_trailing_one_shape():  # tests/ut/test_elemwise.py:219-232
    np.random.seed(1)
    x = np.random.normal(0, 1, [16000, 39, 1]).astype(np.float32)
    y = np.random.normal(0, 1, [16000, 39, 1]).astype(np.float32)
    run_parity(lambda k, a, b: k.mul(a, b), [x, y], golden=x * y)


def test_pow():  # tests/ut/test_elemwise.py:235-279
    a = np.array([-2, -3, -4, 0, -2, 9], np.float32)
    b = np.array([1, 2, 3, 0, 0.5, 0.5], np.float32)
    run_parity(lambda k, p, q: k.pow(p, q), [a, b], golden=np.array([-2, 9, -64, 1, np.nan, 3], np.float32))
    rng = np.random.default_rng(5)
    x = rng.uniform(-5, 5, [32, 64]).astype(np.float32)
    e = rng.integers(0, 6, [32, 64]).astype(np.float32)
    run_parity(lambda k, p, q: k.pow(p, q), [x, e], golden=np.power(x, e), eps=1e-4)
    z = np.abs(rng.normal(0, 1, [32, 1024]) - 2).astype(np.float32)
    for s in (0, 1.2, 5, -7, -3):
        run_parity(lambda k, p: k.add(k.pow(p, s), 2.0), [z], golden=np.power(z, np.float32(s)) + 2, eps=2e-5)
    run_parity(lambda k, p: k.pow(0.91, p), [z], golden=np.power(np.float32(0.91), z))


@pytest.mark.parametrize("dt,eps", [(np.float16, 1e-3), (np.float32, 1e-5)])
def test_rsqrt(dt, eps):  # tests/ut/test_elemwise.py:282-292
    x = np.random.default_rng(6).uniform(0.01, 1, [32, 32]).astype(dt)
    run_parity(lambda k, a: k.reciprocal(k.sqrt(a)), [x], golden=1 / np.sqrt(x), eps=eps)


def test_int32():  # tests/ut/test_elemwise.py:295-428
    rng = np.random.default_rng(7)
    x = rng.integers(-2 ** 30, 2 ** 30, [32, 1024]).astype(np.int32)
    y = rng.integers(-2 ** 30, 2 ** 30, [32, 1024]).astype(np.int32)
    with np.errstate(over="ignore"):
        gold = [x + y, x - y, x * y, np.maximum(x, y), np.minimum(x, y), x + np.int32(11111), x * np.int32(11111),
                np.maximum(x, np.int32(11111)), np.abs(x), np.int32(11111) - x]
    run_parity(lambda k, a, b: [k.add(a, b), k.sub(a, b), k.mul(a, b), k.maximum(a, b), k.minimum(a, b), k.add(a, 11111),
                                k.mul(a, 11111), k.maximum(a, 11111), k.abs(a), k.sub(11111, a)], [x, y], golden=gold)


@pytest.mark.parametrize("shape", [(32, 32), (3145728,)])
@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_round_family(shape, dt):  # tests/ut/test_elemwise.py:456-468
    x = np.random.default_rng(8).normal(-10, 10, shape).astype(dt)
    run_parity(lambda k, a: [k.round(a), k.ceil(a), k.floor(a), k.trunc(a)], [x],
               golden=[np.round(x), np.ceil(x), np.floor(x), np.trunc(x)], eps=0)


def test_casts():  # tests/ut/test_cast.py:26-165
    rng = np.random.default_rng(9)
    h = rng.normal(0, 10, [32, 1000]).astype(np.float16)
    f = rng.normal(0, 10, [32, 1000]).astype(np.float32)
    i = rng.integers(-2000, 2000, [32, 1000]).astype(np.int32)
    b = rng.choice([True, False], [32, 1000])
    run_parity(lambda k, a: [k.cast(a, "float32"), k.cast(a, "int32"), k.cast(a, "bool"), k.cast(a, "bfloat16")], [h],
               golden=[h.astype(np.float32), h.astype(np.int32), h != 0, None], eps=0)
    run_parity(lambda k, a: [k.cast(a, "float16"), k.cast(a, "int32"), k.cast(a, "bool")], [f],
               golden=[f.astype(np.float16), f.astype(np.int32), f != 0], eps=0)
    run_parity(lambda k, a: [k.cast(a, "float32"), k.cast(a, "float16"), k.cast(a, "bool")], [i],
               golden=[i.astype(np.float32), i.astype(np.float16), i != 0], eps=0)
    run_parity(lambda k, a: [k.cast(a, "float32"), k.cast(a, "float16"), k.cast(a, "int32")], [b],
               golden=[b.astype(np.float32), b.astype(np.float16), b.astype(np.int32)], eps=0)
    # bf16 <-> fp32 and arithmetic on bf16 (tests/ut/test_cast.py:41-51)
    outs = run_parity(lambda k, a: [k.cast(a, "bfloat16"), k.cast(k.add(k.cast(a, "bfloat16"), k.cast(a, "bfloat16")), "float32")], [f], eps=0)
    u = f.view(np.uint32).astype(np.uint64)
    bf = (((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)
    assert np.array_equal(outs[0], bf)
    # chained casts and casts mixed with arithmetic
    run_parity(lambda k, a: k.cast(k.cast(k.add(k.cast(a, "float32"), 0.5), "int32"), "float16"), [h],
               golden=(h.astype(np.float32) + np.float32(0.5)).astype(np.int32).astype(np.float16), eps=0)


def test_float_to_int_beyond_the_range_saturates():
    # src/vm_gpu.cu:299-301 on the reference's device: the nearest end of the range, 0 for NaN
    edge = np.tile(np.array([np.inf, -np.inf, np.nan, 3e9, -3e9, 2147483648.0, 2147483520.0, -2147483648.0, -2147483904.0,
                             1.9, -1.9, -0.0], np.float32), 100)
    want = np.tile(np.array([2 ** 31 - 1, -2 ** 31, 0, 2 ** 31 - 1, -2 ** 31, 2 ** 31 - 1, 2147483520, -2 ** 31, -2 ** 31, 1, -1, 0],
                            np.int64).astype(np.int32), 100)
    half = np.tile(np.array([np.inf, -np.inf, np.nan, 65504.0, -1.5], np.float16), 100)
    want_half = np.tile(np.array([2 ** 31 - 1, -2 ** 31, 0, 65504, -1], np.int64).astype(np.int32), 100)
    run_parity(lambda k, a, h: [k.cast(a, "int32"), k.cast(h, "int32"), k.cast(k.mul(a, 1.0), "int32")], [edge, half],
               golden=[want, want_half, want], golden_eps=0)


@pytest.mark.parametrize("shape", [(32, 32), (1024, 32), (1024, 2000)])
@pytest.mark.parametrize("dt", [np.int32, np.float32, np.float16, np.bool_])
def test_compare(shape, dt):  # tests/ut/test_cmp.py:24-170
    rng = np.random.default_rng(shape[1])
    if dt == np.bool_:
        x, y = rng.choice([True, False], shape), rng.choice([True, False], shape)
    elif dt == np.int32:
        x, y = rng.integers(-5, 5, shape).astype(dt), rng.integers(-5, 5, shape).astype(dt)
    else:
        x, y = rng.integers(-3, 3, shape).astype(dt) * dt(0.5), rng.integers(-3, 3, shape).astype(dt) * dt(0.5)
    run_parity(lambda k, a, b: [k.equal(a, b), k.less(a, b), k.greater(a, b), k.less_equal(a, b), k.greater_equal(a, b), k.not_equal(a, b)],
               [x, y], golden=[x == y, x < y, x > y, x <= y, x >= y, x != y])
    if dt != np.bool_:
        s = 1 if dt == np.int32 else 0.5
        run_parity(lambda k, a: [k.equal(a, s), k.less(a, s), k.greater(s, a), k.not_equal(s, a)], [x],
                   golden=[x == s, x < s, s > x, s != x])


def test_compare_bf16():
    rng = np.random.default_rng(10)
    x = (rng.integers(-3, 3, [64, 333]) * 0.5).astype(np.float32)
    y = (rng.integers(-3, 3, [64, 333]) * 0.5).astype(np.float32)
    run_parity(lambda k, a, b: [k.equal(a, b), k.less(a, b), k.greater_equal(a, 0.5)], [x, y], dtypes=["bfloat16", "bfloat16"],
               golden=[x == y, x < y, x >= 0.5])


@pytest.mark.parametrize("shape", [(1024, 32), (13, 131), (16, 11), (3, 3)])
@pytest.mark.parametrize("dt", [np.float32, np.float16, np.int32])
def test_select(shape, dt):  # tests/ut/test_select.py:24-118
    rng = np.random.default_rng(shape[0])
    c = rng.choice([True, False], shape)
    a, b = (rng.normal(0, 10, shape)).astype(dt), (rng.normal(0, 10, shape)).astype(dt)
    run_parity(lambda k, p, q, r: k.select(p, q, r), [c, a, b], golden=np.where(c, a, b), eps=0)
    # broadcast condition, compare-produced condition, scalar branch
    cr = rng.choice([True, False], (shape[0], 1))
    run_parity(lambda k, p, q, r: k.select(k.broadcast(p, list(shape)), q, r), [cr, a, b], golden=np.where(cr, a, b), eps=0)
    run_parity(lambda k, q, r: k.select(k.greater(q, r), q, k.full(1, list(shape), {np.float32: "float32", np.float16: "float16", np.int32: "int32"}[dt])),
               [a, b], golden=np.where(a > b, a, dt(1)), eps=0)


def test_select_bool_values():
    rng = np.random.default_rng(12)
    c, a, b = (rng.choice([True, False], (16, 11)) for _ in range(3))
    run_parity(lambda k, p, q, r: k.select(p, q, r), [c, a, b], golden=np.where(c, a, b))


def test_composite_gelu_tanh():  # tests/ut/test_composite_ops.py:22-71
    np.random.seed(12)
    for dt, eps in [(np.float32, 1e-5), (np.float16, 2e-3)]:
        x = np.random.normal(0, 1, [32, 1024]).astype(dt)

        def tanh(k, v):
            e2 = k.exp(k.mul(v, 2.0))
            return k.div(k.sub(e2, 1.0), k.add(e2, 1.0))

        def gelu(k, v):
            inner = k.mul(k.add(v, k.mul(k.mul(k.mul(v, v), v), 0.044715)), 0.7978845608)
            return k.mul(k.mul(v, 0.5), k.add(tanh(k, inner), 1.0))

        # NumPy golden in the tensor's own precision, operator by operator
        def np_tanh(v):
            e2 = np.exp(v * dt(2.0))
            return (e2 - dt(1.0)) / (e2 + dt(1.0))
        inner = (x + x * x * x * dt(0.044715)) * dt(0.7978845608)
        g = x * dt(0.5) * (np_tanh(inner) + dt(1.0))
        run_parity(lambda k, a: [gelu(k, a), tanh(k, a)], [x], eps=eps, golden=[g, np_tanh(x)], golden_eps=eps * 2)


def test_graph_longer_than_one_program():  # tests/ut/test_eager_fusion.py:551-800 (bytecode beyond 4 KB): cut into several launches
    x = np.random.default_rng(9).normal(0, 1, [64, 48]).astype(np.float32)

    def build(k, a):
        y = a
        for i in range(700):
            y = k.add(y, 0.5) if i % 2 else k.mul(y, 1.001)
        return y
    want = x.copy()
    for i in range(700):
        want = want + np.float32(0.5) if i % 2 else want * np.float32(1.001)
    t = Tester("split")
    out = t.store(build(t, t.load(x)))
    t.run()
    assert 2 <= t.num_launches() <= 10
    assert np.array_equal(t.output(out), want)


def test_tensor_of_more_than_2_32_elements():
    # 5 x 2^30 one-byte elements: device coordinates are 32 bits wide, so the two dims stay apart instead of being
    # merged into one flat axis; the second operand varies along the outer dim only
    pat = np.random.default_rng(0).random(1 << 20) < 0.5
    x = np.tile(pat, 5 * 1024).reshape(5, 1 << 30)
    col = np.array([[True], [False], [True], [True], [False]])
    t = Tester("")
    st = t.store(t.logical_and(t.logical_not(t.load(x)), t.load(col)))
    t.run()
    out = t.output(st)
    assert out.shape == x.shape and out.dtype == np.bool_
    assert np.array_equal(out, ~x & col)
