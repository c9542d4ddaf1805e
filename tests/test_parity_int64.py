"""GPU parity: int64 tensors. The reference lowers them to pairs of int32 tensors, the low and the high words of every
element, in its API layer (src/dvm.cc:478-760: add, sub and the compares with carries and borrows, select, broadcast,
fills, casts), and so does this backend (`Builder::{Add64,Sub64,Compare64,ToInt64,FromInt64}` in host/dvm_api.cc; the
words of a Load are two strided views of its buffer, a Store writes its two inputs through strides). The cases follow
the reference's own int64 tests (tests/ut/test_elemwise.py:189-395, test_cmp.py:175-245, test_select.py:120-173,
test_broadcast.py:99-180, test_view_sch.py:248-262), which run on its Ascend backend only; expectations are NumPy's
int64 arithmetic, bit for bit."""
import numpy as np
import pytest

from dvm_amd import DataType
from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu

BIG = 0x2000000000  # 2^37, the range of the reference's tests


def _rand(rng, shape, lim=BIG):
    return rng.integers(-lim, lim, size=shape, dtype=np.int64)


def _edges():
    # words whose sum or difference carries, borrows, wraps, and the ends of the range
    lo = np.array([0, 1, -1, 0xffffffff, 0x80000000, 0x7fffffff, 0x100000000, -0x100000000, (1 << 32) | 5, -((1 << 32) | 6),
                   np.iinfo(np.int64).min, np.iinfo(np.int64).max, 0x7fffffffffffffff - 1, -0x80000000, 0xfffffffe, 2], dtype=np.int64)
    return lo


def _run(build):
    t = Tester("split")
    outs = build(t)
    t.run()
    return [t.output(o) for o in outs], t


@pytest.mark.parametrize("op,fn", [("add", np.add), ("sub", np.subtract)])
def test_add_sub(op, fn):
    rng = np.random.default_rng(1)
    a, b = _rand(rng, [320, 1024]), _rand(rng, [320, 1024])
    e = _edges()
    a[0, :256] = np.repeat(e, 16)
    b[0, :256] = np.tile(e, 16)
    with np.errstate(over="ignore"):
        want = fn(a, b)
    (got,), t = _run(lambda t: [t.store(getattr(t, op)(t.load(a), t.load(b)))])
    assert got.dtype == np.int64 and np.array_equal(got, want)
    assert t.num_launches() == 1, t.das()


@pytest.mark.parametrize("op,fn", [("add", np.add), ("sub", np.subtract)])
@pytest.mark.parametrize("scalar", [7, -3, 0x1234567890, -0x1fffffffff, 0xffffffff, -(1 << 32)])
@pytest.mark.parametrize("scalar_left", [False, True])
def test_add_sub_scalar(op, fn, scalar, scalar_left):
    rng = np.random.default_rng(2)
    a = _rand(rng, [33, 517])
    a.reshape(-1)[:16] = _edges()
    with np.errstate(over="ignore"):
        want = fn(np.int64(scalar), a) if scalar_left else fn(a, np.int64(scalar))
    build = (lambda t: [t.store(getattr(t, op)(scalar, t.load(a)))]) if scalar_left else (lambda t: [t.store(getattr(t, op)(t.load(a), scalar))])
    (got,), _ = _run(build)
    assert np.array_equal(got, want)


def test_scalar_reference_is_read_at_every_code_generation():
    # tests/ut/test_elemwise.py:344-361: a dynamic shape and an int64 scalar that change between runs of one kernel
    rng = np.random.default_rng(3)
    t = Tester("split:dyn")
    x = t.load([-1], "int64")
    s = t.scalar(DataType.int64)
    y = t.store(t.add(x, s))
    z = t.store(t.full(s, [5], "int64"))
    for n, v in ((100, 0x300000001), (17, -5), (4000, -(1 << 40) + 3)):
        a = _rand(rng, [n])
        t.input(x, a)
        t.input(s, v)
        t.run()
        assert np.array_equal(t.output(y), a + np.int64(v))
        assert np.array_equal(t.output(z), np.full([5], v, np.int64))


CMPS = [("equal", np.equal), ("not_equal", np.not_equal), ("greater", np.greater), ("greater_equal", np.greater_equal),
        ("less", np.less), ("less_equal", np.less_equal)]


@pytest.mark.parametrize("op,fn", CMPS)
def test_compare(op, fn):
    rng = np.random.default_rng(4)
    a, b = _rand(rng, [200, 1000]), _rand(rng, [200, 1000])
    b[::3] = a[::3]                      # equal elements
    b[1::7] = a[1::7] ^ 1                # equal high words, low words one apart
    b[2::11] = a[2::11] ^ (1 << 31)      # the low words' top bit decides: unsigned compare
    e = _edges()
    a[0, :256] = np.repeat(e, 16)
    b[0, :256] = np.tile(e, 16)
    (got,), _ = _run(lambda t: [t.store(getattr(t, op)(t.load(a), t.load(b)))])
    assert got.dtype == np.bool_ and np.array_equal(got, fn(a, b))


@pytest.mark.parametrize("op,fn", CMPS)
@pytest.mark.parametrize("lhs_shape,rhs_shape", [((1, 10, 1, 50), (7, 1, 20, 1)), ((64, 1), (1, 300))])
def test_compare_broadcast(op, fn, lhs_shape, rhs_shape):
    rng = np.random.default_rng(5)
    a, b = _rand(rng, lhs_shape, 1 << 33), _rand(rng, rhs_shape, 1 << 33)
    (got,), _ = _run(lambda t: [t.store(getattr(t, op)(t.load(a), t.load(b)))])
    assert np.array_equal(got, fn(a, b))


@pytest.mark.parametrize("op,fn", CMPS)
@pytest.mark.parametrize("scalar_left", [False, True])
def test_compare_scalar(op, fn, scalar_left):
    rng = np.random.default_rng(6)
    a = _rand(rng, [80, 1000])
    v = 0x123456789
    a[0, :50] = v
    want = fn(np.int64(v), a) if scalar_left else fn(a, np.int64(v))
    build = (lambda t: [t.store(getattr(t, op)(v, t.load(a)))]) if scalar_left else (lambda t: [t.store(getattr(t, op)(t.load(a), v))])
    (got,), _ = _run(build)
    assert np.array_equal(got, want)


def test_select():
    rng = np.random.default_rng(7)
    shape = (13, 131)
    a, b, c, d = (_rand(rng, shape, 1 << 40) for _ in range(4))
    (got,), _ = _run(lambda t: [t.store(t.select(t.greater(t.load(a), t.load(b)), t.load(c), t.load(d)))])
    assert np.array_equal(got, np.where(a > b, c, d))
    # boundary patterns under a bool mask from memory
    e = _edges()
    cond = (np.arange(16) % 3 == 0)
    (got,), _ = _run(lambda t: [t.store(t.select(t.load(cond), t.load(e), t.load(e[::-1].copy())))])
    assert np.array_equal(got, np.where(cond, e, e[::-1]))


def test_select_broadcast():
    rng = np.random.default_rng(8)
    a, b = _rand(rng, (1, 10, 1, 1, 50), 1 << 40), _rand(rng, (1, 1, 20, 30, 1), 1 << 40)
    c, d = _rand(rng, (7, 1, 1, 1, 50), 1 << 40), _rand(rng, (1, 1, 1, 30, 1), 1 << 40)
    (got,), _ = _run(lambda t: [t.store(t.select(t.greater(t.load(a), t.load(b)), t.load(c), t.load(d)))])
    assert np.array_equal(got, np.where(a > b, c, d))


@pytest.mark.parametrize("src,dst", [((1, 300), (40, 300)), ((64, 1), (64, 100)), ((5, 1, 7), (5, 9, 7)), ((1,), (33,))])
def test_broadcast_and_fill(src, dst):
    rng = np.random.default_rng(9)
    a = rng.integers(0x10000000, BIG, size=src, dtype=np.int64)
    (b, f), _ = _run(lambda t: [t.store(t.broadcast(t.load(a), list(dst))), t.store(t.full(-0x1ffffffff7, list(dst), "int64"))])
    assert np.array_equal(b, np.broadcast_to(a, dst)) and np.array_equal(f, np.full(dst, -0x1ffffffff7, np.int64))


def test_casts():
    rng = np.random.default_rng(10)
    s32 = rng.integers(-(1 << 31), (1 << 31) - 1, size=[4096], dtype=np.int64).astype(np.int32)
    s32[:4] = [0, -1, np.iinfo(np.int32).min, np.iinfo(np.int32).max]
    f32 = (rng.standard_normal([4096]) * 2.0 ** rng.integers(0, 61, [4096])).astype(np.float32)
    f32[:8] = [0.0, -0.0, 0.99, -0.99, 4294967296.0, -4294967296.0, 2147483648.0, -2147483649.0]
    f16 = (rng.standard_normal([4096]) * 300).astype(np.float16)
    s64 = _rand(rng, [4096], 1 << 46)
    s64[:16] = _edges()
    small = _rand(rng, [4096], 1 << 24)   # exactly representable in fp32
    outs, _ = _run(lambda t: [t.store(t.cast(t.load(s32), "int64")), t.store(t.cast(t.load(f32), "int64")), t.store(t.cast(t.load(f16), "int64")),
                              t.store(t.cast(t.load(s64), "int32")), t.store(t.cast(t.load(small), "float32")), t.store(t.cast(t.load(s64), "bool")),
                              t.store(t.cast(t.cast(t.load(s64), "int32"), "int64"))])
    assert np.array_equal(outs[0], s32.astype(np.int64))
    assert np.array_equal(outs[1], f32.astype(np.int64))      # truncation toward zero, |x| < 2^63
    assert np.array_equal(outs[2], f16.astype(np.int64))
    assert np.array_equal(outs[3], s64.astype(np.int32))      # the low word
    assert np.array_equal(outs[4], small.astype(np.float32))
    assert np.array_equal(outs[5], s64 != 0)
    assert np.array_equal(outs[6], s64.astype(np.int32).astype(np.int64))


def test_cast_to_float_beyond_24_bits_is_within_a_unit_in_the_last_place():
    rng = np.random.default_rng(11)
    s64 = _rand(rng, [8192], 1 << 62)
    (got,), _ = _run(lambda t: [t.store(t.cast(t.load(s64), "float32"))])
    want = s64.astype(np.float32)
    assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= np.spacing(np.abs(want)).astype(np.float64))


def test_views_and_layout_operators():
    rng = np.random.default_rng(12)
    a = _rand(rng, [6, 20, 16])
    b = _rand(rng, [6, 20, 16])

    def build(t):
        la, lb = t.load(a), t.load(b)
        s = t.add(la, lb)
        return [t.store(t.reshape(s, [120, 16])), t.store(t.permute(s, [2, 0, 1])), t.store(t.slice_dim(s, 1, 3, 11)),
                t.store(t.copy(la)), t.store(t.concat([la, s], 2)), t.store(la)]

    (r, p, sl, c, cat, ident), _ = _run(build)
    s = a + b
    assert np.array_equal(r, s.reshape(120, 16)) and np.array_equal(p, s.transpose(2, 0, 1)) and np.array_equal(sl, s[:, 3:11])
    assert np.array_equal(c, a) and np.array_equal(cat, np.concatenate([a, s], 2)) and np.array_equal(ident, a)


def test_strided_load_and_result_feeding_another_launch():
    # an int64 load through a stride list (every second row of a wider buffer), and an int64 value that crosses launches:
    # its words are two int32 values in the workspace
    rng = np.random.default_rng(13)
    buf = _rand(rng, [64, 40])
    x32 = rng.standard_normal([32, 24], dtype=np.float32)

    def build(t):
        v = t.view_load([32, 24], [80, 1], buf, offset=8)     # rows 0, 2, 4, ..; columns 8..31
        y = t.add(v, 0x100000001)
        rowmax = t.max(t.load(x32), (1,), True)                # a reduce: the pointwise part behind it is another sweep
        pick = t.select(t.greater(t.load(x32), t.sub(rowmax, 1.0)), y, t.sub(y, y))
        return [t.store(pick), t.store(y)]

    (pick, y), _ = _run(build)
    want_y = buf[::2, 8:32] + np.int64(0x100000001)
    assert np.array_equal(y, want_y)
    assert np.array_equal(pick, np.where(x32 > x32.max(1, keepdims=True) - 1.0, want_y, 0))


def test_what_int64_does_not_have():
    t = Tester("split")
    x = t.load(np.zeros([8], np.int64))
    for build in (lambda: t.mul(x, x), lambda: t.abs(x), lambda: t.sum(x, (0,), True), lambda: t.add(x, t.load(np.zeros([8], np.int32)))):
        with pytest.raises(RuntimeError):
            build()
