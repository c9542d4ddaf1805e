"""GPU parity: max / min reduces over the reference's shape list, and run-to-run reproducibility.

Restates tests/ut/test_reduce.py:84-133 (sum / min / max over shapes that exercised tiling bugs there),
:136-172 (tails), :175-276 (deterministic mode: two runs give the same bits) and :311-341. NumPy golden at
the reference's tolerance (1e-4 for sums; max and min exact), the CPU oracle as second opinion. Manual
`tile()` hints of the reference's tests are advice for its tile model and are passed through unchanged."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_parity

pytestmark = pytest.mark.gpu

SHAPES = [([511, 1024], (1,)), ([521, 1024], (1,)), ([35053], (0,)), ([120, 1], (0,)), ([1, 4, 120, 136], (0, 2, 3)),
          ([120, 20, 1], (2,)), ([1, 1, 1, 1, 5, 1, 1, 300, 1, 100], (0, 2, 4, 6, 8)), ([3, 4, 120, 136], (0, 2, 3)),
          ([3, 1280, 2, 2], (0, 2, 3)), ([128, 703], (0,)), ([1, 1024, 14, 14], (0, 2, 3)), ([11, 6000], (0,)),
          ([324, 9, 80], (0, 2))]


@pytest.mark.parametrize("shape,dims", SHAPES)
@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_max_min_shape_list(shape, dims, dt):  # tests/ut/test_reduce.py:84-133
    x = np.random.default_rng(len(shape) * 1000 + shape[0]).normal(-0.5, 0.5, shape).astype(dt)
    run_parity(lambda k, a: [k.max(a, dims, True), k.min(a, dims, True)], [x],
               golden=[np.max(x, dims, keepdims=True), np.min(x, dims, keepdims=True)], eps=0)


def run_twice(build, arrays, goldens, eps=1e-4):
    """Two runs of one compiled kernel must agree bit for bit (tests/ut/test_reduce.py:183-199)."""
    Tester.set_deterministic(True)
    try:
        t = Tester()
        outs = build(t, *[t.load(a) for a in arrays])
        stores = [t.store(o) for o in outs]
        t.run()
        first = [t.output(s).copy() for s in stores]
        t.run()
        second = [t.output(s) for s in stores]
    finally:
        Tester.set_deterministic(False)
    for a, b, g in zip(first, second, goldens):
        assert np.array_equal(a, b), "two runs differ"
        assert np.allclose(b, g, rtol=eps, atol=eps, equal_nan=True)
    return t


@pytest.mark.parametrize("shape,dims,tile_depth", [([400, 4096], (0,), 1), ([40000], (0,), 0), ([65, 40, 4096], (1,), 2),
                                                   ([8, 3, 7, 4, 1024], (1, 3), 3), ([8, 3, 7, 4, 4096], (1, 3), 4),
                                                   ([8, 3, 6, 4, 3, 4, 1024], (1, 3, 5), 5)])
def test_sum_reproducible(shape, dims, tile_depth):  # tests/ut/test_reduce.py:175-201
    a = np.random.default_rng(tile_depth).normal(-0.5, 0.5, shape).astype(np.float32)

    def g(t, x):
        y = t.sum(x, dims, True)
        for i in range(tile_depth):
            t.tile(len(shape) - i - 1, len(shape) - i - 1, shape[i])
        return [y]
    run_twice(g, [a], [np.sum(a.astype(np.float64), dims, keepdims=True)])


def test_two_sums_reproducible():  # tests/ut/test_reduce.py:204-229
    a = np.random.default_rng(21).normal(-0.5, 0.5, [64, 8, 256, 8]).astype(np.float32)
    dims = (0, 2)
    run_twice(lambda t, x: [t.sum(t.mul(x, 1.5), dims, True), t.sum(t.mul(x, 0.8), dims, True)], [a],
              [np.sum(a * np.float32(1.5), dims, keepdims=True), np.sum(a * np.float32(0.8), dims, keepdims=True)])


def test_max_reproducible():  # tests/ut/test_reduce.py:243-258
    a = np.random.default_rng(22).normal(-0.5, 0.5, [65, 40, 4096]).astype(np.float32)
    run_twice(lambda t, x: [t.max(x, (1,), True)], [a], [np.max(a, (1,), keepdims=True)], eps=0)


@pytest.mark.parametrize("dims", [(0,), (0, 2)])
def test_sum_max_min_in_one_kernel_exact(dims):  # tests/ut/test_reduce.py:261-276
    a = np.ones((128, 9, 257), dtype=np.float32)
    a[0] = 2
    a[1] = -2
    run_parity(lambda k, x: [k.sum(x, dims, False), k.max(x, dims, False), k.min(x, dims, False)], [a],
               golden=[np.sum(a, axis=dims), np.max(a, axis=dims), np.min(a, axis=dims)], eps=0)


def test_tails():  # tests/ut/test_reduce.py:136-172
    rng = np.random.default_rng(23)
    a = rng.normal(0, 1, [1949]).astype(np.float32)
    run_parity(lambda k, x: k.sum(x, (0,), True), [a], golden=np.sum(a.astype(np.float64), (0,), keepdims=True), eps=1e-4)
    b = rng.normal(0, 1, [1949, 512]).astype(np.float32)
    run_parity(lambda k, x: k.sum(x, (0,), True), [b], golden=np.sum(b.astype(np.float64), (0,), keepdims=True), eps=1e-4)
    c = np.full([1, 640, 64, 64], 1.0, np.float32)
    run_parity(lambda k, x: k.sum(k.sum(x, [2, 3], True), [0], True), [c], golden=np.full([1, 640, 1, 1], 4096.0, np.float32))


@pytest.mark.parametrize("n", [256 * 50 + 100, 249 * 50 + 223, 501 * 20])
def test_long_vector_sums(n):  # tests/ut/test_reduce.py:311-323
    a = np.random.default_rng(n).normal(0.0, 1.0, [n]).astype(np.float32)
    run_parity(lambda k, x: k.sum(x, (0,), True), [a], golden=np.sum(a.astype(np.float64), (0,), keepdims=True), eps=1e-4)


def test_sum_over_both_axes_of_broadcast_add():  # tests/ut/test_reduce.py:326-341
    rng = np.random.default_rng(24)
    a0, a1 = rng.standard_normal([8002, 2]).astype(np.float32), rng.standard_normal([8002, 1]).astype(np.float32)
    run_parity(lambda k, x0, x1: k.sum(k.add(x0, x1), [0, 1], False), [a0, a1],
               golden=np.sum((a0 + a1).astype(np.float64), axis=(0, 1)), eps=1e-4)


# max / min over int32 tensors compare integers: values above 2^24 (no fp32 holds them), negative values (whose
# bit patterns order backwards as floats) and -1 (the bit pattern of a NaN) come out exact, along the innermost
# axis (one team per output), along an outer axis (lanes own outputs) and with a consumer in the same launch.
INT_SHAPES = [([64, 1000], (1,)), ([1000, 64], (0,)), ([7, 33, 129], (0, 2)), ([3, 40000], (1,)), ([5, 9, 300], (1,)),
              ([200000], (0,))]


@pytest.mark.parametrize("shape,dims", INT_SHAPES)
def test_max_min_int32(shape, dims):
    rng = np.random.default_rng(sum(shape))
    x = rng.integers(-2**31, 2**31 - 1, shape, dtype=np.int64).astype(np.int32)
    x.flat[::97] = -1
    x.flat[5::89] = rng.integers(-40, 40, x.flat[5::89].shape).astype(np.int32)
    mx, mn = np.max(x, dims, keepdims=True), np.min(x, dims, keepdims=True)
    run_parity(lambda k, a: [k.max(a, dims, True), k.min(a, dims, True), k.sub(a, k.max(a, dims, True))], [x],
               golden=[mx, mn, x - mx], eps=0)  # the subtraction wraps in int32, as NumPy's does


def test_max_min_int32_small_negative():
    x = -np.arange(1, 4097, dtype=np.int32).reshape(4, 1024)
    run_parity(lambda k, a: [k.max(a, (1,), False), k.min(a, (0,), False)], [x],
               golden=[np.max(x, 1), np.min(x, 0)], eps=0)
