"""GPU parity: the remaining gpu-marked element-wise cases of tests/ut/test_elemwise.py of the reference, with
their exact shapes: power by tensors, by integer scalars (lowered to a multiply chain whose length the
reference's test pins), by a scalar base; long one-dimensional tensors; logical operators on bools."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_pow_special_values(dt):  # tests/ut/test_elemwise.py:234-246
    a, b = np.array([-2, -3, -4, 0, -2, 9]).astype(dt), np.array([1, 2, 3, 0, 0.5, 0.5]).astype(dt)
    run_graph("", lambda k: [(k.store(k.pow(k.load(a), k.load(b))), np.array([-2, 9, -64, 1, np.nan, 3]).astype(dt), None)])


@pytest.mark.parametrize("dt", [np.float16, np.float32])
@pytest.mark.parametrize("shape", [(1024, 32), (13, 131), (16, 11), (3, 3)])
def test_pow_tensor_exponent(dt, shape):  # :249-264
    rng = np.random.default_rng(shape[1])
    a, b = (10 * rng.random(shape) - 5).astype(dt), rng.integers(0, 6, shape).astype(dt)
    with np.errstate(over="ignore"):
        gold = np.power(a, b)
    run_graph("", lambda k: [(k.store(k.copy(k.pow(k.copy(k.load(a)), k.copy(k.load(b))))), gold, 2e-3 if dt == np.float16 else 1e-5)])


@pytest.mark.parametrize("shape", [(1024, 32), (13, 131)])
@pytest.mark.parametrize("exponent", [0.0, 1.2, 5.0, -7.0, -3.0])
def test_pow_scalar_exponent(shape, exponent):  # :267-279
    a = np.abs(np.random.default_rng(int(exponent * 10) % 7).normal(0, 1, shape).astype(np.float32) - 2)
    run_graph("", lambda k: [(k.store(k.copy(k.add(k.pow(k.load(a), exponent), 2))), np.power(a, np.float32(exponent)) + 2, 2e-5)])


@pytest.mark.parametrize("num,muls", [(3, 2), (10, 4), (-8, 3), (11, 5), (15, 6), (20, 5)])
def test_pow_integer_scalar_is_a_multiply_chain(num, muls):  # :432-441
    arg = np.random.default_rng(abs(num)).random([1024]).astype(np.float32) + np.float32(0.05)
    t = run_graph("", lambda k: [(k.store(k.pow(k.load(arg), num)), np.power(arg, num), 1e-5 if num > 0 else None)], oracle_eps=1e-5)
    assert t.das().count("Mul.fp32") == muls


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_pow_scalar_base(dt):  # :444-453
    a = np.random.default_rng(1).normal(0, 1, (1024, 32)).astype(dt)
    run_graph("", lambda k: [(k.store(k.pow(0.91, k.load(a))), np.power(0.91, a.astype(np.float64)).astype(dt), 1e-3 if dt == np.float16 else 1e-5)])


@pytest.mark.parametrize("dt", [np.float16, np.float32])
def test_long_and_tiny_tensors(dt):  # :160-183, :218-231, :204-215
    a = np.full([32 * 64 * 257], 0.5, dt)
    run_graph("", lambda k: [(k.store(k.add(k.load(a), 0.1)), dt(0.6), None)])
    p, q = np.full([1], 0.4, dt), np.full([1], 0.2, dt)
    run_graph("", lambda k: [(k.store(k.sub(k.load(p), k.load(q))), dt(0.2), None)])
    rng = np.random.default_rng(1)
    a0, a1 = rng.normal(0, 1, [16000, 39, 1]).astype(dt), rng.normal(0, 1, [16000, 39, 1]).astype(dt)
    run_graph("", lambda k: [(k.store(k.mul(k.load(a0), k.load(a1))), a0 * a1, None)])
    shape = [2, 3, 4, 5] if dt == np.float16 else [1, 1, 4, 5]
    y = (rng.random(shape) + 0.05).astype(dt)
    run_graph("", lambda k: [(k.store(k.div(k.full(2, shape, dt.__name__), k.load(y))), dt(2) / y, None)])


def test_logical_on_bools():  # :535-545
    rng = np.random.default_rng(2)
    a, b = rng.choice([True, False], [32, 64]), rng.choice([True, False], [32, 64])
    t = run_graph("", lambda k: [(k.store(k.logical_or(k.logical_not(k.load(a)), k.load(b))), np.logical_or(np.logical_not(a), b), 0)])
    assert t.num_launches() == 1
