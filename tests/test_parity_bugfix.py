"""GPU parity: the regression graphs of the reference's tests/st/test_bugfix.py and the graph set of its
tests/fuzz/test_eager_consistent.py (same operators, shapes and input distributions), against NumPy and the
CPU oracle. The fuzz file checks that rebuilding a graph on a reused kernel object gives the same program each
time; that part runs without a GPU (see tests/test_host.py::test_rebuilt_graphs_compile_to_the_same_program)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def test_many_outputs_then_full_reduce():  # tests/st/test_bugfix.py:20-52
    rng = np.random.default_rng(1)
    big, thin = (2, 576, 224, 16, 2), (2, 576, 224, 16, 1)
    a0, a1, a3, a4, a5 = (rng.standard_normal(s, dtype=np.float32) for s in (big, thin, big, thin, big))
    e0 = a0 + a1
    e1 = e0 * a1
    e2 = a3 * e1
    e3 = a4 * a5
    e4 = e2 * e3

    def g(k):
        x0, x1, x3, x4, x5 = (k.load(a) for a in (a0, a1, a3, a4, a5))
        y0 = k.add(x0, x1)
        y1 = k.mul(y0, x1)
        y2 = k.mul(x3, y1)
        y3 = k.mul(x4, x5)
        y4 = k.mul(y2, y3)
        y5 = k.sum(y4, [0, 1, 2, 3, 4], False)
        return [(k.store(y), e, 1e-4) for y, e in ((y0, e0), (y1, e1), (y2, e2), (y3, e3), (y4, e4))] + \
               [(k.store(y5), np.sum(e4.astype(np.float64)), 1e-4 * np.abs(e4).sum() ** 0.5)]
    run_graph("split", g, oracle_eps=1e-3)


def test_select_with_one_element_condition():  # :55-70
    rng = np.random.default_rng(2)
    ax, bx = rng.normal(0, 0.1, [1, 4, 8192, 96]).astype(np.float16), rng.normal(0, 0.1, [1, 4, 8192, 96]).astype(np.float16)
    cx, dx = np.full([1], 0, np.bool_), np.full([1, 4, 8192, 96], 0.1, np.float16)

    def g(k):
        x0 = k.add(k.load(bx), k.load(ax))
        s0 = k.store(x0)
        return [(s0, ax + bx, None), (k.store(k.select(k.load(cx), k.load(dx), x0)), ax + bx, None)]
    run_graph("split", g)


def test_value_used_by_later_and_earlier_operators():  # :73-90
    rng = np.random.default_rng(3)
    a0, a1 = rng.normal(0, 0.1, [2, 4]).astype(np.float32), rng.normal(0, 0.1, [2, 4]).astype(np.float32)
    e4 = np.exp(a1 * np.float32(-1)) + 1
    e5, e6 = e4 / 1, a1 / e4

    def g(k):
        x0, x1 = k.load(a0), k.load(a1)
        x4 = k.add(k.exp(k.mul(x1, -1)), 1)
        x5, x6 = k.div(x4, 1), k.div(x1, x4)
        return [(k.store(k.mul(k.sub(k.add(x5, x6), k.mul(x5, x6)), x0)), ((e5 + e6) - (e5 * e6)) * a0, None)]
    run_graph("eager", g)


def test_tall_reduce_beside_tiny_kernels():  # :93-104
    rng = np.random.default_rng(4)
    big = rng.normal(0, 0.1, [4096, 40000]).astype(np.float32)
    small = [rng.normal(0, 0.1, [8]).astype(np.float32) for _ in range(8)]

    def g(k):
        outs = [(k.store(k.sum(k.load(big), (0,), True)), np.sum(big.astype(np.float64), (0,), keepdims=True), 1e-3)]
        return outs + [(k.store(k.add(k.load(s), 0.1)), s + np.float32(0.1), None) for s in small]
    run_graph("eager", g)


def test_reduces_and_their_consumers_interleaved():  # :107-146
    rng = np.random.default_rng(5)
    a0, a3, a7 = rng.normal(0, 0.1, [512, 3072]).astype(np.float32), rng.normal(0, 0.1, [4, 128, 768]).astype(np.float32), \
        rng.normal(0, 0.1, [4, 128, 768]).astype(np.float32)
    a8 = (np.abs(rng.normal(0, 0.1, [4, 128, 1])) + 0.05).astype(np.float32)
    a15, a18 = rng.normal(0, 0.1, [768]).astype(np.float32), rng.normal(0, 0.1, [4, 128, 768]).astype(np.float32)

    def g(k):
        out = [(k.store(k.sum(k.load(a0), (0,), False)), np.sum(a0, axis=0), 1e-4)]
        x3, x8 = k.load(a3), k.load(a8)
        out.append((k.store(k.sum(x3, (0, 1), False)), np.sum(a3, axis=(0, 1)), 1e-4))
        x11 = k.add(k.add(x3, -1), k.div(k.div(k.load(a7), x8), x8))
        x12 = k.div(x3, x8)
        out.append((k.store(k.sum(x11, (2,), False)), np.sum((a3 + np.float32(-1)) + (a7 / a8) / a8, axis=2), 2e-3))
        x16 = k.add(x12, k.load(a15))
        out.append((k.store(x16), a3 / a8 + a15, 1e-4))
        out.append((k.store(k.sum(k.add(x12, k.load(a18)), (0, 1), False)), np.sum(a3 / a8 + a18, axis=(0, 1)), 1e-3))
        out.append((k.store(k.sum(k.add(x16, -1), (2,), False)), np.sum((a3 / a8 + a15) + np.float32(-1), axis=2), 2e-3))
        return out
    Tester.set_deterministic(True)
    try:
        run_graph("eager:unify_ws", g, oracle_eps=1e-4)
    finally:
        Tester.set_deterministic(False)


def test_fuzz_graph_two_reduces_of_broadcast_products():  # tests/fuzz/test_eager_consistent.py:36-46
    rng = np.random.default_rng(6)
    a0, a1, a3 = rng.normal(0, 1, [1, 32, 1, 44, 80]).astype(np.float32), rng.normal(0, 1, [1, 32, 100, 44, 80]).astype(np.float32), \
        rng.normal(0, 1, [1, 1, 100, 44, 80]).astype(np.float32)

    def g(k):
        x1 = k.load(a1)
        return [(k.store(k.sum(k.mul(k.load(a0), x1), (1,), False)), np.sum(a0 * a1, axis=1), 1e-4),
                (k.store(k.sum(k.mul(k.load(a3), x1), (2,), False)), np.sum(a3 * a1, axis=2), 1e-4)]
    run_graph("eager", g)


def test_fuzz_graph_batchnorm_statistics_update():  # :47-75
    rng = np.random.default_rng(7)
    a0 = np.ones([96], np.float32)
    a2, a4 = rng.normal(0, 1, [96, 128]).astype(np.float32), rng.normal(1, 1, [96, 128]).astype(np.float32) ** 2
    a15, a23 = rng.normal(0, 1, [128]).astype(np.float32), rng.normal(0, 1, [128]).astype(np.float32)
    n = np.float32(96)
    mean, ex2 = np.sum(a2, 0) / n, np.sum(a4, 0) / n
    var = ex2 - mean * mean

    def g(k):
        x1 = k.sum(k.load(a0), (0,), False)
        x6 = k.div(k.sum(k.load(a2), (0,), False), x1)
        s6 = k.store(x6)
        x10 = k.sub(k.div(k.sum(k.load(a4), (0,), False), x1), k.mul(x6, x6))
        s13 = k.store(k.div(k.sqrt(k.add(x10, 1e-05)), 1))
        s18 = k.store(k.add(k.mul(k.load(a15), 0.9), k.mul(x6, 0.1)))
        x22 = k.mul(x10, k.div(x1, k.add(x1, -1)))
        s26 = k.store(k.add(k.mul(k.load(a23), 0.9), k.mul(x22, 0.1)))
        return [(s6, mean, 1e-4), (s13, np.sqrt(var + np.float32(1e-5)), 1e-4), (s18, a15 * np.float32(0.9) + mean * np.float32(0.1), 1e-4),
                (s26, a23 * np.float32(0.9) + (var * (n / (n - 1))) * np.float32(0.1), 1e-4)]
    run_graph("eager", g, oracle_eps=1e-4)


def test_fuzz_graph_bool_and_cast_chains():  # :76-126
    rng = np.random.default_rng(8)
    a0 = rng.normal(50, 80, [24, 88, 160]).astype(np.float32)
    a0[0, 0, :8] = [np.nan, np.inf, -np.inf, 0, 100, -1, 99.5, 1e30]

    def g(k):
        x0 = k.load(a0)
        x3 = k.cast(k.cast(k.less(x0, 0), "float16"), "bool")
        x6 = k.cast(k.cast(k.less(x0, 100), "float16"), "bool")
        x9 = k.logical_or(k.cast(x3, "float16"), k.cast(x6, "float16"))
        x11 = k.cast(k.less(x9, 0), "bool")
        x15 = k.cast(k.cast(k.less(k.isfinite(x0), 0), "float16"), "bool")
        x18 = k.add(k.mul(k.cast(x15, "float16"), -1), 1)
        x20 = k.cast(k.less(x18, 0), "bool")
        x23 = k.logical_or(k.cast(x11, "float16"), k.cast(x20, "float16"))
        x25 = k.cast(k.less(x23, 0), "bool")
        x28 = k.add(k.mul(k.cast(x25, "float16"), -1), 1)
        x30 = k.cast(k.less(x28, 0), "bool")
        x33 = k.mul(x0, k.cast(k.cast(x30, "float16"), "float32"))
        x36 = k.mul(k.cast(k.cast(x25, "float16"), "float32"), 100)
        return [(k.store(k.add(x33, x36)), None, None)]
    run_graph("eager", g)
    b0 = rng.normal(1, 2, [60, 288, 112]).astype(np.float32)
    run_graph("eager", lambda k: [(k.store(k.cast(k.cast(k.cast(k.cast(k.less(k.load(b0), 1), "float16"), "bool"), "float16"), "float32")),
                                   (b0 < 1).astype(np.float32), 0)])
