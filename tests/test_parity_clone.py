"""GPU parity: cloned kernels, restating the reference's tests/ut/test_clone.py (the speculative-kernel case aside):
a graph copied into a second kernel object runs on new data, new shapes and new axis lists, independent of
the kernel it came from."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def test_clone_vector():  # tests/ut/test_clone.py:21-35
    rng = np.random.default_rng(1)
    a = rng.normal(0, 1, [10, 512]).astype(np.float32)
    t = Tester()
    ax = t.load(a)
    out = t.store_expect(t.sum(t.add(ax, 0.01), [0], True), np.sum(a + np.float32(0.01), (0,), keepdims=True), 1e-4)
    assert t.run_check()
    t2 = Tester()
    ax2, out2 = t2.clone(t, [ax, out])
    a2 = rng.normal(0, 1, [10, 512]).astype(np.float32)
    t2.input(ax2, a2)
    t2.run()
    assert t2.check(out2, np.sum(a2 + np.float32(0.01), (0,), keepdims=True), 1e-4)
    t.run()  # the original still computes its own result
    assert t.check(out, np.sum(a + np.float32(0.01), (0,), keepdims=True), 1e-4)


def test_clone_vector_dyn():  # :36-56
    rng = np.random.default_rng(2)
    t = Tester("vector:dyn")
    ax = t.load([], "float32")
    dims = t.int_array()
    out = t.store(t.sum(t.add(ax, 0.01), dims, True))
    a = rng.normal(0, 1, [10, 512]).astype(np.float32)
    t.input(ax, a)
    dims.update([0])
    t.run()
    assert t.check(out, np.sum(a + np.float32(0.01), (0,), keepdims=True), 1e-4)
    t2 = Tester("vector:dyn")
    ax2, out2, dims2 = t2.clone(t, [ax, out, dims])
    a2 = rng.normal(0, 1, [64, 800]).astype(np.float32)
    t2.input(ax2, a2)
    dims2.update([1])
    t2.run()
    assert t2.check(out2, np.sum(a2 + np.float32(0.01), (1,), keepdims=True), 1e-4)
    t.run()  # the original kept its own shape and axes
    assert t.check(out, np.sum(a + np.float32(0.01), (0,), keepdims=True), 1e-4)


@pytest.mark.parametrize("mode", ["mix", "mix:dyn"])
def test_clone_mix(mode):  # :73-91
    rng = np.random.default_rng(3)
    g0, g1 = rng.normal(0, 0.01, [1024, 1024]).astype(np.float16), rng.normal(0, 0.01, [1024, 1536]).astype(np.float16)
    expect = np.matmul(g0.astype(np.float32), g1.astype(np.float32)).astype(np.float16) + g1
    t = Tester(mode)
    a, b = t.load(g0), t.load(g1)
    out = t.store_expect(t.add(t.matmul(a, b, False, False), b), expect)
    assert t.run_check()
    t2 = Tester(mode)
    a2, b2, out2 = t2.clone(t, [a, b, out])
    t2.input(a2, g0)
    t2.input(b2, g1)
    t2.run()
    assert t2.check(out2, expect)


def test_clone_split_dyn():  # :92-126
    rng = np.random.default_rng(4)
    t = Tester("split:dyn")
    a, b = t.load([], "float16"), t.load([], "float16")
    dims = t.int_array()
    out = t.store(t.mul(t.sum(t.cast(t.matmul(t.mul(a, 0.8), b, False, False), "float32"), dims, True), 0.5))

    def expect(ax, bx, d):
        e = np.matmul((ax * np.float16(0.8)).astype(np.float32), bx.astype(np.float32)).astype(np.float16)
        return np.sum(e.astype(np.float32), d, keepdims=True) * 0.5
    ax, bx = rng.normal(0, 0.1, [512, 1024]).astype(np.float16), rng.normal(0, 0.1, [1024, 1024]).astype(np.float16)
    t.input(a, ax)
    t.input(b, bx)
    dims.update([0])
    t.run()
    assert t.check(out, expect(ax, bx, (0,)), 2e-3)
    t2 = Tester("split:dyn")
    a2, b2, out2, dims2 = t2.clone(t, [a, b, out, dims])
    ax, bx = rng.normal(0, 0.1, [1024, 1024]).astype(np.float16), rng.normal(0, 0.1, [1024, 768]).astype(np.float16)
    t2.input(a2, ax)
    t2.input(b2, bx)
    dims2.update([1])
    t2.run()
    assert t2.check(out2, expect(ax, bx, (1,)), 2e-3)
