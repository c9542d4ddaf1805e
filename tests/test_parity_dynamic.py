"""GPU parity: dynamic shapes, restating tests/ut/test_dynamic_shape.py of the reference: one kernel object, built
once with `-1` extents and with axis / shape lists held by reference, is run on a series of shapes (ranks change
between runs too). NumPy expectations and tolerances as there."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def test_reshape_by_reference():  # tests/ut/test_dynamic_shape.py:20-38
    t = Tester("vector:dyn")
    x, y = t.load([-1], "float32"), t.load([-1], "float32")
    ref = t.int_array()
    out = t.store(t.add(t.reshape(x, ref), y))
    rng = np.random.default_rng(1)
    for xs, rs, ys in [[[10], [2, 5], [2, 5]], [[20, 40], [800, 1], [800, 16]], [[2, 40], [1, 80, 1], [10, 80, 32]]]:
        xd, yd = rng.normal(0, 1, xs).astype(np.float32), rng.normal(0, 1, ys).astype(np.float32)
        t.input(x, xd)
        t.input(y, yd)
        ref.update(rs)
        t.run()
        assert t.check(out, xd.reshape(rs) + yd)


def test_implicit_broadcast():  # :39-57
    t = Tester("vector:dyn")
    x, y = t.load([-1], "float32"), t.load([-1], "float32")
    out = t.store(t.mul(t.add(x, 0.15), y))
    for xs, ys in [[[1000], [1000]], [[500, 1], [500, 1024]], [[500, 1], [1, 1024]], [[4, 1, 12, 1], [4, 32, 12, 64]]]:
        d1, d2 = np.full(xs, 0.1, np.float32), np.full(ys, 0.4, np.float32)
        t.input(x, d1)
        t.input(y, d2)
        t.run()
        assert t.check(out, (d1 + np.float32(0.15)) * d2)


def test_reduce_axes_by_reference():  # :58-71
    t = Tester("vector:dyn")
    x = t.load([-1], "float32")
    dims = t.int_array()
    out = t.store(t.sum(x, dims, True))
    rng = np.random.default_rng(2)
    for xs, ds in [[[10, 64], [1]], [[12, 128], [0, 1]], [[3, 12, 20, 100], [1, 3]]]:
        d1 = rng.normal(0, 1, xs).astype(np.float32)
        t.input(x, d1)
        dims.update(ds)
        t.run()
        assert t.check(out, np.sum(d1, tuple(ds), keepdims=True), 1e-4)


def test_reduce_same_shape_again():  # :72-84
    t = Tester("vector:dyn")
    x = t.load([-1, 2, 4, 3000], "float32")
    out = t.store(t.sum(x, [0, 2], True))
    din = np.random.default_rng(3).normal(0, 1, [2, 2, 4, 3000]).astype(np.float32)
    for _ in range(3):
        t.input(x, din)
        t.run()
        assert t.check(out, np.sum(din, (0, 2), keepdims=True), 1e-4)


def test_cast_add_cast_reduce():  # :85-100
    t = Tester("vector:dyn")
    a = t.load([3, 1280, -1, -1], "float32")
    out = t.store(t.sum(t.cast(t.add(t.cast(a, "float16"), 0.1), "float32"), [0, 2, 3], True))
    rng = np.random.default_rng(4)
    for shape in [[3, 1280, 38, 36], [3, 1280, 44, 22]]:
        ax = rng.normal(0, 0.1, shape).astype(np.float32)
        t.input(a, ax)
        t.run()
        assert t.check(out, np.sum((ax.astype(np.float16) + np.float16(0.1)).astype(np.float32), (0, 2, 3), keepdims=True), 1e-4)


def test_broadcast_shape_by_reference():  # :101-116
    t = Tester("vector:dyn")
    x = t.load([-1], "float32")
    shape = t.int_array()
    out = t.store(t.mul(t.broadcast(x, shape), t.full(0.2, shape, "float32")))
    for xs, bs in [[[1], [10, 100]], [[1, 4, 1], [8, 4, 40]]]:
        xd = np.full(xs, 0.1, np.float32)
        t.input(x, xd)
        shape.update(bs)
        t.run()
        assert t.check(out, np.broadcast_to(xd, bs) * np.float32(0.2))
