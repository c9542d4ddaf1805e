"""GPU parity: "split" kernels (the kernel type the headline configs use), restating the reference's
tests/ut/test_split_graph.py: static and dynamic shapes, unified workspace, matmul with producers and consumers
on either side of the cuts. NumPy expectations and tolerances as there; the CPU oracle as second opinion where
it finishes in seconds."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["split", "split:unify_ws", "split:dyn", "split:dyn,unify_ws"])
def test_long_chain_two_inputs(mode):  # tests/ut/test_split_graph.py:20-39: 200 adds, run on two inputs
    ax = np.random.default_rng(1).normal(0, 0.1, [512, 512]).astype(np.float32)
    bx = np.full([1, 512], 0.01, np.float32)
    t = Tester(mode)
    a, b = t.load([512, 512], "float32"), t.load([1, 512], "float32")
    x = a
    for _ in range(200):
        x = t.add(x, b)
    out = t.store(x)
    for offset in (0.0, 0.1):
        data = ax + np.float32(offset)
        t.input(a, data)
        t.input(b, bx)
        t.run()
        assert t.check(out, data + 0.01 * 200, 1e-4)


@pytest.mark.parametrize("mode", ["split", "split:unify_ws"])
def test_static_vector_graph(mode):  # :40-59
    rng = np.random.default_rng(2)
    a, b = rng.normal(0, 0.1, [10, 4096]).astype(np.float16), rng.normal(0, 0.1, [10, 4096]).astype(np.float32)
    r0 = np.sum((a + np.float16(0.1)).astype(np.float32), (0,), keepdims=True)

    def g(k):
        x = k.add(k.load(a), 0.1)
        s0 = k.store(x)
        x0 = k.sum(k.cast(x, "float32"), (0,), True)
        out1 = k.mul(k.cast(x0, "float16"), 1.5)
        s2 = k.store(k.add(x0, k.load(b)))
        return [(s0, a + np.float16(0.1), None), (s2, r0 + b, None), (k.store(out1), r0.astype(np.float16) * np.float16(1.5), None)]
    run_graph(mode, g)


@pytest.mark.parametrize("mode", ["split", "split:unify_ws"])
def test_static_matmul_with_bias(mode):  # :60-77
    rng = np.random.default_rng(3)
    xd, yd, bd = rng.normal(0, 0.1, [1000, 3333]).astype(np.float16), rng.normal(0, 0.1, [3333, 1024]).astype(np.float16), \
        rng.normal(0, 0.1, [1024]).astype(np.float16)
    res = np.matmul((xd * np.float16(0.5)).astype(np.float32), yd.astype(np.float32)).astype(np.float16) + bd + np.float16(0.1)
    run_graph(mode, lambda k: [(k.store(k.add(k.matmul(k.mul(k.load(xd), 0.5), k.load(yd), False, False, k.load(bd)), 0.1)), res, 2e-3)],
              oracle=mode == "split", oracle_eps=2e-3)


@pytest.mark.parametrize("mode", ["split:dyn", "split:dyn,unify_ws"])
def test_dynamic_vector_graph(mode):  # :78-103
    t = Tester(mode)
    x, y = t.load([-1], "float16"), t.load([-1], "float16")
    ref = t.int_array()
    out = t.store(t.mul(t.cast(t.sum(t.cast(t.add(x, y), "float32"), ref, True), "float16"), 1.5))
    rng = np.random.default_rng(4)
    for s1, s2, dims in [[[10, 4096], [10, 4096], (0,)], [[100, 1], [100, 4096], (1,)], [[16, 4, 128], [16, 1, 128], (2,)]]:
        xd, yd = rng.normal(0, 0.1, s1).astype(np.float16), rng.normal(0, 0.1, s2).astype(np.float16)
        t.input(x, xd)
        t.input(y, yd)
        ref.update(dims)
        t.run()
        assert t.check(out, np.sum((xd + yd).astype(np.float32), dims, keepdims=True).astype(np.float16) * np.float16(1.5))


@pytest.mark.parametrize("mode", ["split:dyn", "split:dyn,unify_ws"])
def test_dynamic_matmul(mode):  # :104-129
    t = Tester(mode)
    x, y, z = t.load([-1, -1], "float16"), t.load([-1, -1], "float16"), t.load([-1, -1], "float16")
    out = t.store(t.add(t.matmul(t.mul(x, 0.5), y, False, False), z))
    rng = np.random.default_rng(5)
    for xs, ys, zs in [[[256, 128], [128, 256], [256, 256]], [[444, 3333], [3333, 1111], [1, 1111]], [[256, 128], [128, 512], [256, 1]]]:
        xd, yd, zd = (rng.normal(0, 0.1, s).astype(np.float16) for s in (xs, ys, zs))
        t.input(x, xd)
        t.input(y, yd)
        t.input(z, zd)
        t.run()
        assert t.check(out, np.matmul((xd * np.float16(0.5)).astype(np.float32), yd.astype(np.float32)).astype(np.float16) + zd, 2e-3)


def test_dynamic_column_sums():  # :130-143
    t = Tester("split:dyn")
    x = t.load([-1, -1], "float32")
    out = t.store(t.sum(x, [0], True))
    rng = np.random.default_rng(6)
    for shape in [[4, 4096], [4, 512]]:
        xd = rng.normal(0, 0.1, shape).astype(np.float32)
        t.input(x, xd)
        t.run()
        assert t.check(out, np.sum(xd, (0,), keepdims=True))


@pytest.mark.parametrize("x_shape,y_shape,mode", [([1024, 2048], [2048, 2048], "split"), ([1024, 2048], [2048, 2048], "split:dyn"),
                                                  ([1024, 40960], [40960, 4096], "split")])
def test_matmul_stored_and_used(x_shape, y_shape, mode):  # :144-165
    np.random.seed(7)
    xd, yd = Tester.fast_random_normal(0, 0.1, x_shape).astype(np.float16), Tester.fast_random_normal(0, 0.1, y_shape).astype(np.float16)
    res = np.matmul((xd * np.float16(0.5)).astype(np.float32), yd.astype(np.float32)).astype(np.float16)

    def g(k):
        x = k.matmul(k.mul(k.load(xd), 0.5), k.load(yd), False, False)
        s0 = k.store(x)
        return [(s0, res, 2e-3), (k.store(k.add(x, 0.1)), res + np.float16(0.1), 2e-3)]
    # rows of fast_random_normal are equal, sums over k = 40960 reach hundreds: tolerance relative to that, as np.allclose's rtol does
    run_graph(mode, g, oracle=mode == "split:dyn", oracle_eps=2e-3)  # the scalar oracle takes 18 s on this size: once is enough


@pytest.mark.parametrize("mode", ["split:unify_ws", "split:dyn,unify_ws"])
def test_workspace_alignment(mode):  # :166-183: odd sizes between the launches
    np.random.seed(8)
    bd = np.random.normal(0, 0.1, [1979]).astype(np.float32)
    xd, yd = Tester.fast_random_normal(0, 0.1, [4, 512]).astype(np.float16), Tester.fast_random_normal(0, 0.1, [512, 1979]).astype(np.float16)
    res = np.matmul(xd.astype(np.float32), yd.astype(np.float32)).astype(np.float16) + bd.astype(np.float16) + np.float16(0.1)
    run_graph(mode, lambda k: [(k.store(k.add(k.matmul(k.load(xd), k.load(yd), False, False, k.cast(k.load(bd), "float16")), 0.1)), res, 2e-3)],
              oracle_eps=2e-3)


def test_unified_workspace_reduce():  # :184-195
    a = np.random.default_rng(9).normal(-0.5, 0.5, [30, 4000]).astype(np.float32)
    Tester.set_deterministic(True)
    try:
        run_graph("split:unify_ws", lambda k: [(k.store(k.add(k.sum(k.mul(k.load(a), 1.5), (0,), True), 0.1)),
                                                np.sum(a * np.float32(1.5), (0,), keepdims=True) + 0.1, None)])
    finally:
        Tester.set_deterministic(False)


def test_tuning_switch_is_accepted():  # :196-209: the reference tunes tiles online; here the switch changes nothing
    rng = np.random.default_rng(10)
    a, b = rng.normal(0, 0.01, [4096, 4096]).astype(np.float16), rng.normal(0, 0.01, [4096, 4096]).astype(np.float16)
    Tester.set_online_tuning(True)
    try:
        run_graph("split", lambda k: [(k.store(k.matmul(k.load(a), k.load(b), False, False)),
                                       np.matmul(a.astype(np.float32), b.astype(np.float32)), 1e-3)], oracle=False)
    finally:
        Tester.set_online_tuning(False)
