"""Committed golden vectors (tests/golden/vectors.npz, written by tests/golden/make_golden.py from the NumPy
formulas of the reference's tests): the CPU oracle must reproduce them (no GPU), and so must the HIP path."""
import math
import os

import numpy as np
import pytest

from oracle.oracle import OracleKernel

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"))


def _bn(k, x, g, b):
    inv = 1.0 / (x_shape(x)[0] * x_shape(x)[2] * x_shape(x)[3])
    mean = k.mul(k.sum(x, (0, 2, 3), True), inv)
    var = k.sub(k.mul(k.sum(k.mul(x, x), (0, 2, 3), True), inv), k.mul(mean, mean))
    scale = k.div(g, k.sqrt(k.add(var, 1e-5)))
    return k.add(k.mul(x, scale), k.sub(b, k.mul(mean, scale)))


def x_shape(x):
    return x.a.shape if hasattr(x, "a") else x.shape()


def _attention(k, q, kk, v):
    x = k.cast(k.mul(k.matmul(q, kk, False, True), 1.0 / math.sqrt(8)), "float32")
    x = k.sub(x, k.max(x, (1,), True))
    e = k.exp(x)
    return k.matmul(k.cast(k.div(e, k.sum(e, (1,), True)), "float16"), v, False, False)


def _silu(k, a, b, bias):
    h = k.add(k.cast(k.matmul(a, b, False, False), "float32"), bias)
    return k.cast(k.div(h, k.add(k.exp(k.mul(h, -1.0)), 1.0)), "float16")


# (name of the expected vector, input vector names, load dtypes, graph, tolerance: 0 = bit exact)
CASES = [
    ("ew_add", ["ew_a", "ew_b"], None, lambda k, a, b: k.add(a, b), 0), ("ew_sub", ["ew_a", "ew_b"], None, lambda k, a, b: k.sub(a, b), 0),
    ("ew_mul", ["ew_a", "ew_b"], None, lambda k, a, b: k.mul(a, b), 0), ("ew_div", ["ew_a", "ew_b"], None, lambda k, a, b: k.div(a, b), 1e-6),
    ("ew_max", ["ew_a", "ew_b"], None, lambda k, a, b: k.maximum(a, b), 0), ("ew_min", ["ew_a", "ew_b"], None, lambda k, a, b: k.minimum(a, b), 0),
    ("ew_abs", ["ew_a"], None, lambda k, a: k.abs(a), 0), ("ew_exp", ["ew_a"], None, lambda k, a: k.exp(a), 1e-5),
    ("ew_sqrt", ["ew_a"], None, lambda k, a: k.sqrt(k.abs(a)), 1e-6), ("ew_log", ["ew_a"], None, lambda k, a: k.log(k.add(k.abs(a), 1.0)), 1e-5),
    ("ew_round", ["ew_a"], None, lambda k, a: k.round(a), 0), ("ew_floor", ["ew_a"], None, lambda k, a: k.floor(a), 0),
    ("ew_ceil", ["ew_a"], None, lambda k, a: k.ceil(a), 0), ("ew_trunc", ["ew_a"], None, lambda k, a: k.trunc(a), 0),
    ("ew_gt", ["ew_a", "ew_b"], None, lambda k, a, b: k.greater(a, b), 0), ("ew_eq", ["ew_a"], None, lambda k, a: k.equal(a, a), 0),
    ("ew_select", ["ew_a", "ew_b"], None, lambda k, a, b: k.select(k.greater(a, b), a, b), 0),
    ("i_add", ["i_a", "i_b"], None, lambda k, a, b: k.add(a, b), 0), ("i_mul", ["i_a", "i_b"], None, lambda k, a, b: k.mul(a, b), 0),
    ("i_abs", ["i_a"], None, lambda k, a: k.abs(a), 0), ("h_mul", ["h_a"], None, lambda k, a: k.mul(a, a), 0),
    ("c_to_bf16", ["c_f32"], None, lambda k, a: k.cast(a, "bfloat16"), 0), ("c_to_f16", ["c_f32"], None, lambda k, a: k.cast(a, "float16"), 0),
    ("c_to_i32", ["c_f32"], None, lambda k, a: k.cast(a, "int32"), 0),
    ("r_sum_last", ["r_x"], None, lambda k, a: k.sum(a, (3,), True), 1e-5), ("r_sum_023", ["r_x"], None, lambda k, a: k.sum(a, (0, 2, 3), True), 1e-5),
    ("r_max_1", ["r_x"], None, lambda k, a: k.max(a, (1,), False), 0), ("r_min_13", ["r_x"], None, lambda k, a: k.min(a, (1, 3), False), 0),
    ("b_add", ["r_x", "b_row"], None, lambda k, a, b: k.add(a, b), 0),
    ("bn_y", ["bn_x", "bn_g", "bn_b"], None, _bn, 1e-5),
    ("mm_c", ["mm_a", "mm_b"], None, lambda k, a, b: k.matmul(a, b, False, False), 1e-3),
    ("mm_silu", ["mm_a", "mm_b", "mm_bias"], None, _silu, 2e-3),
    ("at_o", ["at_q", "at_k", "at_v"], None, _attention, 1e-2),
]


def _check(name, got, eps):
    want = V[name]
    assert got.shape == want.shape, (name, got.shape, want.shape)
    if eps == 0:
        assert np.array_equal(got, want), name
    else:
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=eps, atol=eps), name


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_oracle_reproduces_golden(case):
    name, ins, _, graph, eps = case
    o = OracleKernel()
    got = o.output(o.store(graph(o, *[o.load(V[n]) for n in ins])))
    if name == "c_to_bf16":
        got = got.astype(np.float32)
    _check(name, got, eps)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_hip_reproduces_golden(case):
    from dvm_amd.tester import Tester
    name, ins, _, graph, eps = case
    t = Tester("mix" if name.startswith(("mm_", "at_")) else "split")
    out = t.store(graph(t, *[t.load(V[n]) for n in ins]))
    t.run()
    got = t.output(out)
    if name == "c_to_bf16":
        got = Tester.convert_from_bf16(got)
    _check(name, got, eps)
