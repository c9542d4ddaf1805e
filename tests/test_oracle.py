"""Pins the CPU oracle (oracle/dvm_oracle.c + oracle/oracle.py) without a GPU.

Checks, chosen so that a plausible mistake (wrong rounding mode, dropped NaN case,
wrong operand order, truncation vs rounding) fails one of them:
  * fp16 codec: every one of the 65536 bit patterns round-trips through fp32 exactly as
    numpy.float16 does; random and tie fp32 values round like numpy (round to nearest even);
  * bf16 codec: closed form on ties, carries into the exponent, inf, NaN (host form -> 0x7fc0,
    src/dvm.cc:173-186), and the bf16 truncation trick of the reference's tester (python/dvm/tester.py:93-99);
  * the constants of the reference's own tests: 0.5 / 0.4 element-wise table (tests/ut/test_elemwise.py:24-54),
    0.1 + 0.3 (examples/01_add.py:27-34), pow special values [-2, 9, -64, 1, nan, 3]
    (tests/ut/test_elemwise.py:235-246), sum of 64 x 0.01 = 0.64 (tests/ut/test_reduce.py:74-83),
    add->sum 40.96 (tests/ut/test_reduce.py:232-241);
  * int32 wrap-around like NumPy (tests/ut/test_elemwise.py:295-428), float -> int32 truncation,
    round half to even (tests/ut/test_elemwise.py:456-468);
  * lowering rules against NumPy: logical ops over bool / fp16 / fp32, compares of mixed dtypes,
    scalar-left sub / div, pow by integer and scalar ** x;
  * sum against float64 NumPy sums, max / min exact, matmul against np.matmul on fp32 copies
    (tests/ut/test_matmul.py:34-36), batch-norm restatement against the float64 closed form.
"""
import numpy as np
import pytest

from oracle import oracle as ora
from oracle.oracle import OracleKernel


def test_f16_all_bit_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = ora.f16_bits_to_f32(bits)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    back = ora.f32_to_f16_bits(ref)
    nan = np.isnan(ref)
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.all((back[nan] & 0x7c00) == 0x7c00) and np.all((back[nan] & 0x3ff) != 0)


def test_f32_to_f16_rounding_matches_numpy():
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.normal(0, 1, 200000), rng.normal(0, 1e-5, 50000), rng.normal(0, 3e4, 50000),
        np.array([65504.0, 65519.9, 65520.0, 65536.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, -0.0, np.inf, -np.inf]),
    ]).astype(np.float32)
    # exact ties between neighbouring halves
    h = rng.integers(0x0001, 0x7bff, 20000).astype(np.uint16)
    a = h.view(np.float16).astype(np.float32)
    b = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    x = np.concatenate([x, (a + b) / 2, -(a + b) / 2]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(ora.f32_to_f16_bits(x), want)


def test_bf16_codec():
    def bits(v):
        return int(ora.f32_to_bf16_bits(np.array([v], np.float32))[0])
    assert bits(1.0) == 0x3f80
    assert bits(np.float32(1.0) + np.float32(2 ** -8)) == 0x3f80       # tie -> even (down)
    assert bits(np.float32(1.0) + np.float32(3 * 2 ** -8)) == 0x3f82   # tie -> even (up)
    assert bits(np.float32(1.0) + np.float32(2 ** -8) + np.float32(2 ** -20)) == 0x3f81
    assert bits(np.array([0x3fffffff], np.uint32).view(np.float32)[0]) == 0x4000  # carry into the exponent
    assert bits(np.inf) == 0x7f80 and bits(-np.inf) == 0xff80
    assert bits(np.nan) == 0x7fc0
    x = np.random.default_rng(3).normal(0, 10, 100000).astype(np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    want = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(ora.f32_to_bf16_bits(x), want)
    # values that are already bf16 (the reference tester's truncation) convert exactly
    t = (x.view(np.uint32) & 0xFFFF0000).view(np.float32)
    assert np.array_equal(ora.bf16_bits_to_f32(ora.f32_to_bf16_bits(t)), t)


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_elementwise_constants(dt):
    k = OracleKernel()
    x = np.full([32, 1024], 0.5, dt)
    y = np.full([32, 1024], 0.4, dt)
    a, b = k.load(x), k.load(y)
    eps = 1e-3 if dt == np.float16 else 1e-6
    for got, want in [(k.sqrt(a), np.sqrt(x)), (k.abs(a), np.abs(x)), (k.log(a), np.log(x)), (k.exp(a), np.exp(x)),
                      (k.reciprocal(a), np.reciprocal(x)), (k.add(a, b), x + y), (k.sub(a, b), x - y),
                      (k.div(a, b), x / y), (k.mul(a, b), x * y), (k.maximum(a, b), np.maximum(x, y)),
                      (k.minimum(a, b), np.minimum(x, y))]:
        assert np.allclose(k.output(got).astype(np.float32), want.astype(np.float32), rtol=eps, atol=eps)
    # fp16 arithmetic is "fp32 op, round once": identical to numpy's half arithmetic, bit for bit
    if dt == np.float16:
        rng = np.random.default_rng(5)
        p, q = rng.normal(0, 1, 4096).astype(dt), rng.normal(0, 1, 4096).astype(dt)
        for f, g in [(k.add, np.add), (k.sub, np.subtract), (k.mul, np.multiply), (k.div, np.divide)]:
            assert np.array_equal(k.output(f(k.load(p), k.load(q))).view(np.uint16), g(p, q).view(np.uint16))


def test_add_example_and_reduce_constants():
    k = OracleKernel()
    x, y = np.full([32, 32], 0.1, np.float32), np.full([32, 32], 0.3, np.float32)
    assert np.array_equal(k.output(k.add(k.load(x), k.load(y))), x + y)
    z = k.load(np.full([64, 1001], 0.01, np.float32))
    assert np.allclose(k.output(k.sum(z, (0,), False)), 0.64, rtol=1e-6)
    a = k.load(np.full([32, 2048], 0.01, np.float32))
    assert np.allclose(k.output(k.sum(k.add(a, a), (1,), True)), 40.96, rtol=1e-6)


def test_pow_special_values():
    k = OracleKernel()
    a = np.array([-2, -3, -4, 0, -2, 9], np.float32)
    b = np.array([1, 2, 3, 0, 0.5, 0.5], np.float32)
    got = k.output(k.pow(k.load(a), k.load(b)))
    assert np.allclose(got, [-2, 9, -64, 1, np.nan, 3], equal_nan=True)
    x = np.abs(np.random.default_rng(1).normal(0, 1, 1000) - 2).astype(np.float32)
    for s in (0, 1.2, 5, -7, -3):
        assert np.allclose(k.output(k.pow(k.load(x), s)), np.power(x, np.float32(s)), rtol=1e-5, atol=1e-5)
    assert np.allclose(k.output(k.pow(0.91, k.load(x))), np.power(np.float32(0.91), x), rtol=1e-5, atol=1e-6)


def test_int32_wraparound_and_casts():
    rng = np.random.default_rng(2)
    x = rng.integers(-2 ** 30, 2 ** 30, [32, 1024]).astype(np.int32)
    y = rng.integers(-2 ** 30, 2 ** 30, [32, 1024]).astype(np.int32)
    k = OracleKernel()
    a, b = k.load(x), k.load(y)
    with np.errstate(over="ignore"):
        assert np.array_equal(k.output(k.add(a, b)), x + y)
        assert np.array_equal(k.output(k.sub(a, b)), x - y)
        assert np.array_equal(k.output(k.mul(a, b)), x * y)
        assert np.array_equal(k.output(k.add(a, 11111)), x + np.int32(11111))
    assert np.array_equal(k.output(k.maximum(a, b)), np.maximum(x, y))
    assert np.array_equal(k.output(k.abs(a)), np.abs(x))
    f = rng.normal(0, 100, 10000).astype(np.float32)
    assert np.array_equal(k.output(k.cast(k.load(f), "int32")), np.trunc(f).astype(np.int32))
    assert np.array_equal(k.output(k.cast(k.load(x[0]), "float32")), x[0].astype(np.float32))
    h = rng.normal(0, 10, 10000).astype(np.float16)
    assert np.array_equal(k.output(k.cast(k.load(h), "int32")), np.trunc(h.astype(np.float32)).astype(np.int32))
    # beyond the range of int32 the conversion saturates and NaN gives 0: what the reference's C cast
    # (src/vm_gpu.cu:299-301) means on its device (PTX cvt.rzi.s32.f32); known answers, not a host cast (undefined there)
    edge = np.array([np.inf, -np.inf, np.nan, 3e9, -3e9, 2147483648.0, 2147483520.0, -2147483648.0, -2147483904.0,
                     1.9, -1.9, -0.0], np.float32)
    want = np.array([2 ** 31 - 1, -2 ** 31, 0, 2 ** 31 - 1, -2 ** 31, 2 ** 31 - 1, 2147483520, -2 ** 31, -2 ** 31, 1, -1, 0],
                    np.int64).astype(np.int32)
    assert np.array_equal(k.output(k.cast(k.load(edge), "int32")), want)
    assert np.array_equal(k.output(k.cast(k.load(np.array([np.inf, -np.inf, np.nan, 65504.0], np.float16)), "int32")),
                          np.array([2 ** 31 - 1, -2 ** 31, 0, 65504], np.int64).astype(np.int32))
    r = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 2.4999, 3.5001], np.float32)
    assert np.array_equal(k.output(k.round(k.load(r))), np.round(r))
    assert np.array_equal(k.output(k.floor(k.load(f))), np.floor(f))
    assert np.array_equal(k.output(k.ceil(k.load(f))), np.ceil(f))
    assert np.array_equal(k.output(k.trunc(k.load(f))), np.trunc(f))


@pytest.mark.parametrize("dt", [np.bool_, np.float16, np.float32])
def test_logical_rules(dt):
    rng = np.random.default_rng(4)
    x = rng.choice([True, False], [128, 777]).astype(dt)
    y = rng.choice([True, False], [128, 777]).astype(dt)
    k = OracleKernel()
    a, b = k.load(x), k.load(y)
    assert np.array_equal(k.output(k.logical_and(a, b)).astype(bool), np.logical_and(x, y))
    assert np.array_equal(k.output(k.logical_or(a, b)).astype(bool), np.logical_or(x, y))
    assert np.array_equal(k.output(k.logical_not(a)).astype(bool), np.logical_not(x))


def test_compare_select_scalar_rules():
    rng = np.random.default_rng(6)
    xi = rng.integers(-1024, 1024, [128, 77]).astype(np.int32)
    yi = rng.integers(-1024, 1024, [128, 77]).astype(np.int32)
    xf = rng.normal(0, 1, [128, 77]).astype(np.float32)
    yf = rng.normal(0, 1, [128, 77]).astype(np.float32)
    k = OracleKernel()
    g = k.greater(k.load(xi), k.load(yi))
    l = k.less(k.load(xf), k.load(yf))
    assert g.t == ora.BOOL and np.array_equal(k.output(g), xi > yi)
    assert np.array_equal(k.output(k.logical_and(g, l)), np.logical_and(xi > yi, xf < yf))
    assert np.array_equal(k.output(k.select(l, k.load(xf), k.load(yf))), np.where(xf < yf, xf, yf))
    assert np.array_equal(k.output(k.greater_equal(0.25, k.load(xf))), 0.25 >= xf)
    assert np.array_equal(k.output(k.sub(0.1, k.load(xf))), xf * np.float32(-1.0) + np.float32(0.1))
    assert np.array_equal(k.output(k.sub(k.load(xf), 0.1)), xf + np.float32(-0.1))
    assert np.array_equal(k.output(k.div(2.0, k.load(xf))), np.float32(2.0) / xf)
    hf = xf.astype(np.float16)
    assert np.array_equal(k.output(k.div(2.0, k.load(hf))).view(np.uint16), (np.float16(2.0) / hf).view(np.uint16))
    assert np.array_equal(k.output(k.isfinite(k.load(np.array([1, np.inf, -np.inf, np.nan], np.float32)))), [1, 0, 0, 0])


def test_reduce_against_float64():
    rng = np.random.default_rng(8)
    x = rng.normal(-0.5, 0.5, [6, 4, 2, 5, 1, 3, 8]).astype(np.float32)
    k = OracleKernel()
    for dims in [(0,), (6,), (1, 3), (0, 2, 5), (0, 1, 2, 3, 4, 5, 6)]:
        for keep in (True, False):
            want = np.sum(x.astype(np.float64), axis=dims, keepdims=keep).astype(np.float32)
            assert np.array_equal(k.output(k.sum(k.load(x), dims, keep)), want)
            assert np.array_equal(k.output(k.max(k.load(x), dims, keep)), np.max(x, axis=dims, keepdims=keep))
            assert np.array_equal(k.output(k.min(k.load(x), dims, keep)), np.min(x, axis=dims, keepdims=keep))
    nanx = np.array([[1.0, np.nan, 3.0], [1.0, 2.0, 3.0]], np.float32)
    assert np.array_equal(k.output(k.max(k.load(nanx), (1,), False)), np.max(nanx, 1), equal_nan=True)


def test_matmul_against_numpy():
    np.random.seed(1)
    for dt, eps in [(np.float16, 1e-3), ("bfloat16", 5e-3)]:
        a = np.random.normal(0, 0.1, (64, 96)).astype(np.float32)
        b = np.random.normal(0, 0.1, (96, 48)).astype(np.float32)
        k = OracleKernel()
        la = k.load(a.astype(np.float16) if dt == np.float16 else a, None if dt == np.float16 else dt)
        lb = k.load(b.astype(np.float16) if dt == np.float16 else b, None if dt == np.float16 else dt)
        want = np.matmul(la.a, lb.a)
        assert np.allclose(k.output(k.matmul(la, lb, False, False)).astype(np.float32), want, rtol=eps, atol=eps)
        lbt = k.load(np.ascontiguousarray(lb.a.T), None if dt == np.float16 else dt) if dt != np.float16 else k.load(np.ascontiguousarray(lb.a.T).astype(np.float16))
        assert np.array_equal(k.output(k.matmul(la, lbt, False, True)), k.output(k.matmul(la, lb, False, False)))
    # an exactly representable case: no tolerance
    a = np.arange(12, dtype=np.float32).reshape(3, 4).astype(np.float16)
    b = np.arange(8, dtype=np.float32).reshape(4, 2).astype(np.float16)
    k = OracleKernel()
    assert np.array_equal(k.output(k.matmul(k.load(a), k.load(b), False, False)), (a.astype(np.float32) @ b.astype(np.float32)).astype(np.float16))


def test_matmul_transposes_and_bias_against_numpy():
    """All four storage layouts and the bias row, on shapes where m, n and k all differ (a transposed index or a
    bias added along the wrong axis changes the result), exactly representable values, so no tolerance."""
    rng = np.random.default_rng(77)
    m, n, kk = 5, 7, 11
    a = rng.integers(-4, 5, (m, kk)).astype(np.float16)
    b = rng.integers(-4, 5, (kk, n)).astype(np.float16)
    bias = rng.integers(-8, 9, (n,)).astype(np.float16)
    want = a.astype(np.float32) @ b.astype(np.float32)
    for ta in (False, True):
        for tb in (False, True):
            k = OracleKernel()
            la = k.load(np.ascontiguousarray(a.T) if ta else a)
            lb = k.load(np.ascontiguousarray(b.T) if tb else b)
            assert np.array_equal(k.output(k.matmul(la, lb, ta, tb)), want.astype(np.float16)), (ta, tb)
            got = k.output(k.matmul(la, lb, ta, tb, k.load(bias)))
            assert np.array_equal(got, (want + bias.astype(np.float32)[None, :]).astype(np.float16)), (ta, tb)
    # batches broadcast like np.matmul; the bias joins the fp32 sum before the one rounding
    a3 = rng.normal(0, 1, (3, 1, m, kk)).astype(np.float16)
    b3 = rng.normal(0, 1, (1, 2, kk, n)).astype(np.float16)
    k = OracleKernel()
    got = k.output(k.matmul(k.load(a3), k.load(b3), False, False, k.load(bias)))
    ref = np.matmul(a3.astype(np.float32), b3.astype(np.float32)) + bias.astype(np.float32)
    assert got.shape == (3, 2, m, n) and np.allclose(got.astype(np.float32), ref, rtol=2e-3, atol=2e-3)
    tiny = np.float16(2.0 ** -12)  # 1 + 2^-12 + 2^-12 rounds to 1 + 2^-10 only if the bias is added before rounding
    k = OracleKernel()
    one = k.load(np.array([[1.0, tiny]], np.float16))
    got = k.output(k.matmul(one, k.load(np.array([[1.0], [1.0]], np.float16)), False, False, k.load(np.array([tiny * 2], np.float16))))
    assert got[0, 0] == np.float16(1.0 + 3 * 2.0 ** -12)  # = nearest fp16 to 1.000732, i.e. 1 + 2^-10


def test_int32_min_compares_and_reduces():
    """int32 minimum, every compare and max / min reduces against NumPy, with values fp32 cannot hold."""
    rng = np.random.default_rng(5)
    x = rng.integers(-2 ** 31, 2 ** 31 - 1, [16, 257], dtype=np.int64).astype(np.int32)
    y = rng.integers(-2 ** 31, 2 ** 31 - 1, [16, 257], dtype=np.int64).astype(np.int32)
    y[::2] = x[::2]                 # equal pairs, so that == / != / <= / >= see both outcomes
    y[1, :] = x[1, :] + 1           # neighbours above 2^24, which fp32 would merge
    k = OracleKernel()
    a, b = k.load(x), k.load(y)
    assert np.array_equal(k.output(k.minimum(a, b)), np.minimum(x, y))
    assert np.array_equal(k.output(k.maximum(a, b)), np.maximum(x, y))
    for name, fn in [("equal", np.equal), ("not_equal", np.not_equal), ("greater", np.greater), ("greater_equal", np.greater_equal),
                     ("less", np.less), ("less_equal", np.less_equal)]:
        got = k.output(getattr(k, name)(a, b))
        assert np.array_equal(got.astype(bool), fn(x, y)), name
        got = k.output(getattr(k, name)(a, 7))
        assert np.array_equal(got.astype(bool), fn(x, np.int32(7))), name + " scalar"
    for dims in [(0,), (1,), (0, 1)]:
        assert np.array_equal(k.output(k.max(a, dims, True)), np.max(x, dims, keepdims=True))
        assert np.array_equal(k.output(k.min(a, dims, False)), np.min(x, dims))


def test_batchnorm_restatement():
    rng = np.random.default_rng(1002)
    x = rng.normal(0, 1, [4, 16, 7, 9]).astype(np.float32)
    g = rng.uniform(0.5, 1.5, [16]).astype(np.float32)
    b = rng.normal(0, 0.1, [16]).astype(np.float32)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean((0, 2, 3), keepdims=True)) / np.sqrt(x64.var((0, 2, 3), keepdims=True) + 1e-5)
    want = want * g[None, :, None, None] + b[None, :, None, None]
    assert np.allclose(ora.batchnorm_nchw(x, g, b, 1e-5), want, rtol=1e-5, atol=1e-5)


def test_view_ops_against_element_loops():
    # The view operators of the oracle (strided loads and stores, slices, permute, split, concat) against plain
    # element-by-element loops over the flat buffer and against the values the reference's own tests expect
    # (tests/ut/test_view.py: every tenth column, a transpose, zero strides, an element offset; tests/ut/test_slice.py:
    # negative and out-of-range bounds), on inputs whose elements are all different.
    k = OracleKernel()
    a = np.arange(6 * 40, dtype=np.float32).reshape(6, 40)
    flat = a.reshape(-1)

    def by_loops(shape, stride, offset=0):
        out = np.zeros(shape, np.float32)
        for idx in np.ndindex(*shape):
            out[idx] = flat[offset + sum(i * s for i, s in zip(idx, stride))]
        return out
    for shape, stride, offset in [([6, 4], [40, 10], 0), ([40, 6], [1, 40], 0), ([3, 5, 8], [80, 0, 2], 7), ([2, 20], [40, 1], 60)]:
        assert np.array_equal(k.output(k.view_load(shape, stride, a, offset)), by_loops(shape, stride, offset))
    assert np.array_equal(k.output(k.view_load([6, 4], [40, 10], a)), a[:, 0:40:10])         # tests/ut/test_view.py:137-144
    assert np.array_equal(k.output(k.view_load([40, 6], [1, 40], a)), a.T)                   # :183-201
    assert np.array_equal(k.output(k.slice_load(a, (1, 3), (4, 20))), a[1:5, 3:23])
    assert np.array_equal(k.output(k.stridedslice_load(a, (-5, 0), (100, 40), (1, 1))), a[-5:100])  # tests/ut/test_slice.py:76-89
    assert np.array_equal(k.output(k.stridedslice_load(a, (1, 2), (-2, 38), (2, 3))), a[1:-2:2, 2:38:3])
    # a strided store: element i, j of the value lands at i * 50 + j * 2 of a zero-filled buffer
    v = k.load(a[:3, :10])
    e = np.zeros([4, 50], np.float32)
    got = k.output(k.view_store_expect(v, [50, 2], e))
    want = np.zeros(200, np.float32)
    for i in range(3):
        for j in range(10):
            want[i * 50 + j * 2] = a[i, j]
    assert np.array_equal(got, want.reshape(4, 50))
    # permute: result dim i is input dim dims[i] (include/dvm.h:428-434 of the reference)
    b = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    p = k.output(k.permute(k.load(b), [2, 0, 1]))
    assert p.shape == (4, 2, 3) and all(p[z, x, y] == b[x, y, z] for x in range(2) for y in range(3) for z in range(4))
    # slices of values, split with a smaller last chunk, concat
    assert np.array_equal(k.output(k.slice(k.load(a), [1, 5], [2, 7])), a[1:3, 5:12])
    assert np.array_equal(k.output(k.slice_dim(k.load(a), 1, 5, -2)), a[:, 5:38])
    parts = k.split(k.load(a), 1, 16, 3)
    assert [k.output(x).shape for x in parts] == [(6, 16), (6, 16), (6, 8)] and np.array_equal(k.output(parts[2]), a[:, 32:])
    c = k.output(k.concat([parts[2], parts[0]], 1))
    assert c.shape == (6, 24) and np.array_equal(c[:, :8], a[:, 32:]) and np.array_equal(c[:, 8:], a[:, :16])


def test_values_of_rank_zero_keep_their_rank():
    # a reduce over every dim without keepdims has rank 0 (src/ops.cc:3080-3117); operators on it keep that rank
    from oracle.oracle import OracleKernel
    k = OracleKernel()
    x = k.load(np.arange(5, dtype=np.float32))
    m = k.max(x, (0,), False)
    y = k.floor(k.add(m, 0.5))
    assert k.output(k.store(m)).shape == () and k.output(k.store(y)).shape == ()
    assert float(k.output(k.store(y))) == 4.0
    assert k.output(k.store(k.add(x, y))).shape == (5,)


def _onehot_by_reference_rule(indices, depth, axis, on_value, off_value):
    """The expectation the reference's own test builds (tests/ut/test_onehot.py:22-38): indices seen as [outer, inner]
    around the new dim, out[x, indices[x, y], y] = on_value in a buffer filled with off_value."""
    axis = axis if axis >= 0 else indices.ndim + axis + 1
    outer = int(np.prod(indices.shape[:axis], dtype=np.int64))
    inner = int(np.prod(indices.shape[axis:], dtype=np.int64))
    ix = indices.reshape(outer, inner)
    out = np.full((outer, depth, inner), off_value, np.int32 if isinstance(on_value, int) else np.float32)
    for x in range(outer):
        for y in range(inner):
            out[x, ix[x, y], y] = on_value
    return out.reshape(indices.shape[:axis] + (depth,) + indices.shape[axis:])


def test_gather_onehot_pad_any_against_numpy_and_the_reference_rule():
    rng = np.random.default_rng(11)
    k = OracleKernel()
    # one_hot against the rule of the reference's test, every axis position, both value classes
    for shape, depth in [((5,), 7), ((4, 6), 5), ((2, 3, 4), 3)]:
        ix = rng.integers(0, depth, shape).astype(np.int32)
        for axis in list(range(len(shape) + 1)) + [-1]:
            got = k.output(k.one_hot(k.load(ix), depth, axis, 2.0, 0.5, "float32"))
            assert np.array_equal(got, _onehot_by_reference_rule(ix, depth, axis, 2.0, 0.5))
            got = k.output(k.one_hot(k.load(ix), depth, axis, 3, -1, "int32"))
            assert got.dtype == np.int32 and np.array_equal(got, _onehot_by_reference_rule(ix, depth, axis, 3, -1))
    # an index outside [0, depth) matches no position; on / off are rounded to the result type
    got = k.output(k.one_hot(k.load(np.array([-1, 0, 9], np.int32)), 4, 1, 1.0, 0.0, "float32"))
    assert np.array_equal(got, np.array([[0, 0, 0, 0], [1, 0, 0, 0], [0, 0, 0, 0]], np.float32))
    got = k.output(k.one_hot(k.load(np.array([1], np.int32)), 2, 0, 0.1, 0.3, "float16"))
    assert got.dtype == np.float16 and np.array_equal(got, np.array([[0.3], [0.1]], np.float16))
    # gathers against NumPy's take / take_along_axis, negative indices included (tests/ut/test_gather_load.py:33-75)
    for src_shape, ix_shape, axis in [((6, 5), (7,), 0), ((3, 8, 4), (2, 5), 1), ((2, 4, 6), (9,), -1), ((2, 3, 5, 4), (3, 2), 2)]:
        x = rng.normal(0, 1, src_shape).astype(np.float32)
        n = src_shape[axis]
        ix = rng.integers(-n, n, ix_shape).astype(np.int32)
        got = k.output(k.gather_load(x, k.global_access(ix), axis=axis, gather_mode=1))
        assert np.array_equal(got, np.take(x, ix, axis=axis))
        along_shape = list(src_shape)
        along_shape[axis] = 3
        ia = rng.integers(-n, n, along_shape).astype(np.int32)
        got = k.output(k.gather_load(x, k.global_access(ia), axis=axis))
        assert np.array_equal(got, np.take_along_axis(x, ia.astype(np.int64), axis=axis))
    # indices past either end are clipped into the axis
    x = np.arange(5, dtype=np.float32)
    got = k.output(k.gather_load(x, k.global_access(np.array([7, -9, 4, -5], np.int32)), axis=0, gather_mode=1))
    assert np.array_equal(got, np.array([4, 0, 4, 0], np.float32))
    # pad_store (src/ops.cc:1399-1412): rows pad elements longer, zeros in the padding
    v = rng.normal(0, 1, (3, 4)).astype(np.float32)
    got = k.output(k.pad_store(k.load(v), 5))
    assert got.shape == (3, 9) and np.array_equal(got[:, :4], v) and not got[:, 4:].any()
    # element_any: 1 when any element of a 0 / 1 mask is set (tests/ut/test_element_any.py:22-50)
    m = np.zeros((9, 9), np.float32)
    assert k.output(k.element_any(k.load(m))).tolist() == [0.0]
    m[3, 7] = 1
    assert k.output(k.element_any(k.load(m))).tolist() == [1.0]


def test_grouped_matmul_against_float64_rule():
    # the reference's own expectation (tests/ut/test_gmm.py:25-76) in float64: per group, rows [lo, hi) of x times
    # matrix g of w (groups of rows), or columns [lo, hi) of x times rows [lo, hi) of w (groups along k), + bias row g
    rng = np.random.default_rng(21)
    k = OracleKernel()
    m, n, kk, g = 37, 24, 50, 4
    x = rng.normal(0, 0.5, (m, kk)).astype(np.float16)
    wm = rng.normal(0, 0.5, (g, kk, n)).astype(np.float16)
    wk = rng.normal(0, 0.5, (kk, n)).astype(np.float16)
    b = rng.normal(0, 0.5, (g, n)).astype(np.float16)
    for bounds, sizes in [([5, 5, 20, 37], False), ([5, 0, 15, 17], True), ([3, 30, 37, 37], False)]:
        ends = np.cumsum(bounds) if sizes else np.array(bounds)
        want = np.zeros((m, n))
        lo = 0
        for i, hi in enumerate(ends):
            want[lo:hi] = x[lo:hi].astype(np.float64) @ wm[i].astype(np.float64) + b[i].astype(np.float64)
            lo = hi
        got = k.output(k.grouped_matmul(k.load(x), k.load(wm), False, False, k.load(b), k.load(np.array(bounds, np.int64)), 0, int(sizes)))
        assert got.dtype == np.float16 and np.allclose(got, want, rtol=2e-3, atol=2e-3)
        # transposed operands give the same product
        got_t = k.output(k.grouped_matmul(k.load(np.ascontiguousarray(x.T)), k.load(np.ascontiguousarray(wm.transpose(0, 2, 1))), True, True,
                                          k.load(b), k.load(np.array(bounds, np.int64)), 0, int(sizes)))
        assert np.array_equal(got_t, got)
    for bounds, sizes in [([0, 7, 7, 50], False), ([10, 0, 25, 15], True)]:
        ends = np.cumsum(bounds) if sizes else np.array(bounds)
        want = np.zeros((g, m, n))
        lo = 0
        for i, hi in enumerate(ends):
            want[i] = x[:, lo:hi].astype(np.float64) @ wk[lo:hi].astype(np.float64) + b[i].astype(np.float64)
            lo = hi
        got = k.output(k.grouped_matmul(k.load(x), k.load(wk), False, False, k.load(b), k.load(np.array(bounds, np.int64)), 2, int(sizes)))
        assert got.shape == (g, m, n) and np.allclose(got, want, rtol=2e-3, atol=2e-3)
    # rows past the last bound are not written (zeros here); bounds past the axis are clipped
    got = k.output(k.grouped_matmul(k.load(x), k.load(wm), False, False, None, k.load(np.array([5, 9, 9, 12], np.int64)), 0))
    assert not got[12:].any() and got[:12].any()
    a = k.output(k.grouped_matmul(k.load(x), k.load(wm), False, False, None, k.load(np.array([5, 9, 20, 99], np.int64)), 0))
    c = k.output(k.grouped_matmul(k.load(x), k.load(wm), False, False, None, k.load(np.array([5, 9, 20, 37], np.int64)), 0))
    assert np.array_equal(a, c)
