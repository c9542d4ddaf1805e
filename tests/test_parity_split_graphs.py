"""GPU parity: the graphs of the reference's tests of its graph-kernel splitter (tests/ut/test_split_sym_graph.py,
kernel type "split:priv1": the flag picks the newer of the reference's two split implementations,
src/dvm.cc:1088-1097, and is accepted here without effect). Values several consumers on both sides of a reduce or
a matmul share, loads shared between stages, a matmul whose right operand also feeds a reduce, dynamic shapes of
different rank. Against the oracle and the NumPy expectations the reference's tests state."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu

KER = "split:priv1"


def test_reduce_over_rows_with_consumers_on_both_sides():
    rng = np.random.default_rng(1)
    a = (rng.standard_normal([10, 4096]) * 0.1).astype(np.float16)
    b = (rng.standard_normal([10, 4096]) * 0.1).astype(np.float32)
    shifted = a + np.float16(0.1)
    col = np.sum(shifted.astype(np.float32), (0,), keepdims=True)

    def build(k):
        x = k.add(k.load(a), 0.1)
        s0 = k.store(x)
        total = k.sum(k.cast(x, "float32"), (0,), True)
        s2 = k.store(k.add(total, k.load(b)))
        s1 = k.store(k.mul(k.cast(total, "float16"), 1.5))
        return [(s0, shifted, None), (s2, col + b, 1e-4), (s1, col.astype(np.float16) * np.float16(1.5), 2e-3)]
    run_graph(KER, build, oracle_eps=2e-3)


def test_scaled_operand_into_a_matmul_with_an_add_behind():
    rng = np.random.default_rng(2)
    xd = (rng.standard_normal([1000, 3333]) * 0.1).astype(np.float16)
    yd = (rng.standard_normal([3333, 1024]) * 0.1).astype(np.float16)
    gold = np.matmul((xd * np.float16(0.5)).astype(np.float32), yd.astype(np.float32)).astype(np.float16) + np.float16(0.1)

    def build(k):
        out = k.add(k.matmul(k.mul(k.load(xd), 0.5), k.load(yd), False, False), 0.1)
        return [(k.store(out), gold, 2e-3)]
    run_graph(KER, build, oracle=False)


def test_reshape_between_two_operators():
    rng = np.random.default_rng(3)
    a = rng.standard_normal([32, 128], dtype=np.float32)

    def build(k):
        r = k.add(k.reshape(k.mul(k.load(a), 0.6), [2, 16, 128]), 0.1)
        return [(k.store(r), (a * np.float32(0.6)).reshape([2, 16, 128]) + np.float32(0.1), None)]
    run_graph(KER, build)


def test_select_of_three_operands_that_all_broadcast():
    rng = np.random.default_rng(4)
    cond = rng.uniform(0, 1, (2, 1, 4)) > 0.5
    lhs = (rng.standard_normal((1, 3, 4)) * 0.1).astype(np.float32)
    rhs = (rng.standard_normal((2, 3, 1)) * 0.1).astype(np.float32)

    def build(k):
        return [(k.store(k.select(k.load(cond), k.load(lhs), k.load(rhs))), np.where(cond, lhs, rhs), 0)]
    run_graph(KER, build)


def test_matmul_and_reduce_share_the_right_operand():
    rng = np.random.default_rng(5)
    kk, n, m = 1024, 1280, 640
    a, c = ((rng.standard_normal((kk, n)) * 0.02).astype(np.float16) for _ in range(2))
    b, d = ((rng.standard_normal((kk, m)) * 0.02).astype(np.float16) for _ in range(2))
    lhs_g, rhs_g = np.maximum(a + c, np.float16(0)), b * d
    bias_g = np.sum(rhs_g.astype(np.float32), axis=0, keepdims=True).astype(np.float16).astype(np.float32)
    gold = np.maximum(np.matmul(lhs_g.T.astype(np.float32), rhs_g.astype(np.float32)) + bias_g, 0) * np.float32(0.5)

    def build(k):
        lhs = k.maximum(k.add(k.load(a), k.load(c)), 0.0)
        rhs = k.mul(k.load(b), k.load(d))
        mm = k.cast(k.matmul(lhs, rhs, True, False), "float32")
        bias = k.cast(k.sum(k.cast(rhs, "float32"), (0,), True), "float16")
        out = k.mul(k.maximum(k.add(mm, k.cast(bias, "float32")), 0.0), 0.5)
        return [(k.store(out), gold, 1e-3)]
    run_graph(KER, build, oracle=False)


def test_gelu_written_out_on_rows_of_five():
    rng = np.random.default_rng(6)
    xd = (rng.standard_normal((768, 5)) * 0.02).astype(np.float32)
    inner = (xd + xd * xd * xd * np.float32(0.044715)) * np.float32(-1.5957691216057308)
    gold = xd / (np.exp(inner) + np.float32(1.0))

    def build(k):
        x = k.load(xd)
        cube = k.mul(k.mul(k.mul(x, x), x), 0.044715)
        e = k.exp(k.mul(k.add(x, cube), -1.5957691216057308))
        return [(k.store(k.div(x, k.add(e, 1.0))), gold, 1e-5)]
    run_graph(KER, build)


def test_layer_norm_backward_piece_with_a_zero_divisor():
    # tests/ut/test_split_sym_graph.py:132-191: a row statistic divided by 2 * sqrt, selected against a constant
    # where the square root is zero, then scaled back over the row
    rng = np.random.default_rng(0)
    big = lambda: (rng.standard_normal((4, 128, 768)) * 0.02).astype(np.float32)  # noqa: E731
    xd, subd, tand, gd, expd = big(), big(), big(), big(), big()
    gamma = (rng.standard_normal((768,)) * 0.02).astype(np.float32)
    root = (1.0 + rng.standard_normal((4, 128, 1)) * 0.02).astype(np.float32)
    root[0, 0, 0] = 0.0
    denom = (1.0 + rng.standard_normal((4, 128, 1)) * 0.02).astype(np.float32)
    zero = np.array(0.0, dtype=np.float32)

    prod = -xd * (gamma * subd / denom / denom)
    row = np.sum(prod, axis=2, keepdims=True)
    two_root = root * np.float32(2.0)
    quotient = np.divide(row, two_root, out=np.zeros_like(row), where=two_root != 0)
    picked = np.where(root > 0, quotient, zero) * np.float32(0.002607561929595828)
    gold = (tand + gd) + picked * subd + expd / np.float32(768.0)

    def build(k):
        x, g, sub = k.load(xd), k.load(gamma), k.load(subd)
        tangents, other, rt, ex, dn, z = k.load(tand), k.load(gd), k.load(root), k.load(expd), k.load(denom), k.load(zero)
        neg = k.mul(x, -1.0)
        scaled = k.mul(g, sub)
        base = k.add(tangents, other)
        two = k.mul(rt, 2.0)
        positive = k.greater(rt, 0.0)
        mean_term = k.div(ex, 768.0)
        total = k.sum(k.mul(neg, k.div(k.div(scaled, dn), dn)), (2,), True)
        where = k.select(positive, k.div(total, two), z)
        out = k.add(k.add(base, k.mul(k.mul(where, 0.002607561929595828), sub)), mean_term)
        return [(k.store(out), gold, 1e-4)]
    run_graph(KER, build, oracle_eps=1e-4)


def test_dynamic_shapes_of_rank_two_and_three():
    t = Tester("split:dyn,priv1")
    x0 = t.load([-1, -2], "float32")
    x1 = t.mul(x0, 0.6)
    x2 = t.load([-3, -1, -2], "float32")
    o1 = t.store(t.add(x1, x2))
    x4 = t.load([-4, -1, -2], "float32")
    o2 = t.store(t.sub(x4, x1))
    t.codegen()
    rng = np.random.default_rng(8)
    for s0, s2, s4 in [([256, 128], [4, 256, 128], [3, 256, 128]), ([10, 32], [20, 10, 32], [40, 10, 32])]:
        a, b, c = ((rng.standard_normal(s) * 0.1).astype(np.float32) for s in (s0, s2, s4))
        t.input(x0, a)
        t.input(x2, b)
        t.input(x4, c)
        t.run()
        assert t.check(o1, a * np.float32(0.6) + b)
        assert t.check(o2, c - a * np.float32(0.6))


def test_two_outputs_of_one_load():
    rng = np.random.default_rng(9)
    xd = (rng.standard_normal([64, 1024]) * 0.1).astype(np.float16)

    def build(k):
        x = k.load(xd)
        return [(k.store(k.add(x, 0.1)), xd + np.float16(0.1), None), (k.store(k.mul(x, 2.0)), xd * np.float16(2.0), None)]
    t = run_graph(KER, build)
    assert t.num_launches() == 1, t.das()
