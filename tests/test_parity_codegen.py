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
