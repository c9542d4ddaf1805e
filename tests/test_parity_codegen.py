"""GPU parity: the code-generation stress cases of the reference's tests/ut/test_codegen.py: several reduces with a
reshape between them, many inputs and outputs in one graph, equal expressions stored several times."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def test_several_reduces_and_a_reshape():  # tests/ut/test_codegen.py:21-44
    rng = np.random.default_rng(0)
    a, b, c, w = (rng.normal(0, 0.5, s).astype(np.float32) for s in [(1, 128, 128), (128, 128), (1, 128, 128), (128,)])
    ea = a + b.reshape(1, 128, 128)

    def g(k):
        x0, x1, x2, x3 = (k.load(d) for d in (a, b, c, w))
        sum_a = k.sum(k.reshape(x0, [128, 128]), [0], True)
        added = k.add(x0, k.reshape(x1, [1, 128, 128]))
        return [(k.store(sum_a), a.reshape(128, 128).sum(axis=0, keepdims=True), 1e-4),
                (k.store(k.sum(added, [0, 1], True)), ea.sum(axis=(0, 1), keepdims=True), 1e-4),
                (k.store(k.sum(k.mul(added, x2), [0, 1], True)), (ea * c).sum(axis=(0, 1), keepdims=True), 1e-4),
                (k.store(k.mul(added, k.broadcast(x3, [1, 128, 128]))), ea * w.reshape(1, 1, 128), 1e-4)]
    Tester.set_deterministic(True)
    try:
        run_graph("vector", g)
    finally:
        Tester.set_deterministic(False)


def test_multi_in_multi_out():  # :45-65
    rng = np.random.default_rng(1)
    a0 = np.abs(rng.normal(0, 1, [8, 32000]).astype(np.float32))
    a1 = np.abs(rng.normal(0, 1, [8, 1]).astype(np.float32)) + np.float32(1e-6)
    a2 = rng.normal(0, 1, [8, 32000]).astype(np.float32)
    e0 = a0 / a1

    def g(k):
        y0 = k.div(k.load(a0), k.load(a1))
        s0 = k.store(y0)
        y4 = k.mul(k.mul(k.log(k.add(y0, 1e-24)), k.load(a2)), -1.0)
        return [(s0, e0, None), (k.store(y4), -(np.log(e0 + np.float32(1e-24)) * a2), 1e-4)]
    with np.errstate(divide="ignore", invalid="ignore"):
        run_graph("", g, oracle_eps=1e-4)


def test_equal_expressions_stored_three_times():  # :66-80
    rng = np.random.default_rng(2)
    a0, a1 = rng.normal(0, 1, [1024, 1024]).astype(np.float32), rng.normal(0, 1, [1024, 1024]).astype(np.float32)

    def g(k):
        x0, x1 = k.load(a0), k.load(a1)
        b, a, f = k.sub(x0, x1), k.sub(x0, x1), k.sub(x1, x0)
        return [(k.store(a), a0 - a1, None), (k.store(f), a1 - a0, None), (k.store(b), a0 - a1, None)]
    run_graph("", g)


def test_seventeen_inputs_sixteen_outputs():  # :81-95
    def g(k):
        x = k.load(np.full([512], 0.1, np.float32))
        loads = [k.load(np.full([512], 0.2, np.float32)) for _ in range(16)]
        out, result = [], np.float32(0.1)
        for i in range(16):
            x = k.add(x, loads[i])
            result = result + np.float32(0.2)
            out.append((k.store(x), result, None))
        return out
    run_graph("", g)


def test_three_stores_of_two_expressions_in_reverse_order():  # tests/ut/test_codegen.py:66-82
    rng = np.random.default_rng(1)
    a0, a1 = rng.standard_normal([1024, 1024], dtype=np.float32), rng.standard_normal([1024, 1024], dtype=np.float32)

    def g(k):
        x0, x1 = k.load(a0), k.load(a1)
        b, a, f = k.sub(x0, x1), k.sub(x0, x1), k.sub(x1, x0)
        return [(k.store(a), a0 - a1, 0), (k.store(f), a1 - a0, 0), (k.store(b), a0 - a1, 0)]
    run_graph("vector", g)


def test_value_with_three_readers_of_different_age():  # tests/ut/test_codegen.py:102-113 (run here, listed there)
    rng = np.random.default_rng(2)
    x = np.abs(rng.standard_normal([32, 1024])).astype(np.float16) + np.float16(0.5)

    def g(k):
        v = k.load(x)
        root, mag = k.sqrt(v), k.abs(v)
        return [(k.store(k.add(k.add(root, mag), k.reciprocal(mag))), np.sqrt(x) + np.abs(x) + np.reciprocal(np.abs(x)), 2e-3)]
    run_graph("vector", g)


def test_tensor_without_elements():  # tests/ut/test_codegen.py:116-138
    t = Tester("vector")
    out = t.store(t.mul(t.load(np.full([10, 0, 2], 0.1, np.float32)), 0.1))
    t.run()
    assert out.shape() == (10, 0, 2) and t.output(out).shape == (10, 0, 2)
    t = Tester("vector")
    out = t.store_expect(t.sum(t.add(t.load(np.full([10, 0, 2], 0.01, np.float32)), 0.1), (1,), True), 0.0)
    assert t.run_check()
    assert out.shape() == (10, 1, 2)


def test_dynamic_load_that_changes_rank_and_loses_its_elements():  # tests/ut/test_codegen.py:141-165
    t = Tester("vector:dyn")
    x1 = t.load([-1], "float32")
    out = t.store(t.sum(t.add(x1, 0.1), (1,), True))
    t.input(x1, np.full([10, 0, 20], 0.01, np.float32))
    t.run()
    assert t.check(out, 0.0) and out.shape() == (10, 1, 20)
    t.input(x1, np.full([0, 10, 20], 0.01, np.float32))
    t.run()
    assert out.shape() == (0, 1, 20)
    t.input(x1, np.full([10, 40, 20], 0.01, np.float32))
    t.run()
    assert t.check(out, (np.float32(0.01) + np.float32(0.1)) * 40) and out.shape() == (10, 1, 20)


def test_dynamic_rows_of_4096_around_a_multiple_of_the_workgroup_count():  # tests/ut/test_dynamic_shape.py:136-162
    t = Tester("vector:dyn")
    p0, p1 = t.load([-1], "float16"), t.load([-1], "float16")
    y0 = t.add(p0, p1)
    out0 = t.store(y0)
    y1 = t.cast(y0, "float32")
    out1 = t.store(y1)
    out2 = t.store(t.sum(t.mul(y1, y1), [2], True))
    np.random.seed(3)
    for rows in (2685, 2686, 2687):
        a = Tester.fast_random_normal(0, 1, [1, rows, 4096]).astype(np.float16)
        b = Tester.fast_random_normal(0, 1, [1, rows, 4096]).astype(np.float16)
        t.input(p0, a)
        t.input(p1, b)
        t.run()
        s = (a + b).astype(np.float32)
        assert t.check(out0, a + b) and t.check(out1, s)
        assert t.check(out2, np.sum(s * s, (2,), keepdims=True), 1e-4)


@pytest.mark.parametrize("ker", ["vector", "split", "eager"])
@pytest.mark.parametrize("shape", [[0], [0, 5], [5, 0], [3, 0, 4], [0, 3, 4], [3, 4, 0], [2, 0, 0], [1, 0, 1]])
def test_an_extent_of_zero_anywhere(ker, shape):
    # elementwise, casts, reduces over each axis (the sum of nothing is 0), layout operators, a broadcast partner,
    # and a second output that does have elements, in one kernel each
    rng = np.random.default_rng(len(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    partner = rng.standard_normal([1 if d == 0 else d for d in shape]).astype(np.float32)
    full = rng.standard_normal([4, 8]).astype(np.float32)
    graphs = [lambda k: [k.exp(k.load(x))], lambda k: [k.add(k.mul(k.load(x), 2.0), 1.0)],
              lambda k: [k.cast(k.load(x), "float16"), k.cast(k.load(x), "int32")],
              lambda k: [k.sum(k.load(x), tuple(range(len(shape))), True)],
              lambda k: [k.add(k.load(x), k.load(partner))],
              lambda k: [k.exp(k.load(x)), k.add(k.load(full), 1.0)],
              lambda k: [k.select(k.greater(k.load(x), 0.0), k.load(x), k.mul(k.load(x), 2.0))]]
    for ax in range(len(shape)):
        graphs += [lambda k, ax=ax: [k.sum(k.load(x), (ax,), True)], lambda k, ax=ax: [k.sum(k.load(x), (ax,), False)]]
    if len(shape) >= 2:
        graphs.append(lambda k: [k.add(k.permute(k.load(x), list(range(len(shape)))[::-1]), 1.0)])
        flat = [int(np.prod(shape[:-1])), shape[-1]] if shape[-1] != 0 else [0]
        graphs.append(lambda k: [k.mul(k.reshape(k.load(x), flat), 2.0)])
    for g in graphs:
        run_graph(ker, lambda k, g=g: [(k.store(v), None, None) for v in g(k)])
