"""GPU parity: compares and selects, restating the gpu-marked cases of tests/ut/test_cmp.py and test_select.py of
the reference with their exact shapes and input recipes (NaN rows, bool scalars, full-range int32, operands
that broadcast along the innermost axis over 100000 rows, five-dimensional broadcasts, 0-d operands). Results
are bools or copies of inputs, so everything is compared exactly, with NumPy and with the CPU oracle."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu

OPS = [("equal", np.equal), ("less", np.less), ("greater", np.greater), ("greater_equal", np.greater_equal),
       ("less_equal", np.less_equal), ("not_equal", np.not_equal)]


@pytest.mark.parametrize("shape", [(32, 32), (1024, 32), (1024, 2000)])
@pytest.mark.parametrize("dt", [np.int32, np.float32, np.float16, np.bool_])
def test_cmp(shape, dt):  # tests/ut/test_cmp.py:21-42, all six operators in one graph
    rng = np.random.default_rng(shape[1] + np.dtype(dt).itemsize)
    a, b = rng.integers(0, 1024, shape).astype(dt), rng.integers(0, 1024, shape).astype(dt)
    if dt in (np.float32, np.float16):
        a[0] = np.nan
        b[0] = np.nan

    def g(k):
        x, y = k.copy(k.load(a)), k.copy(k.load(b))
        return [(k.store(k.copy(getattr(k, name)(x, y))), fn(a, b), 0) for name, fn in OPS]
    with np.errstate(invalid="ignore"):
        run_graph("split", g)


@pytest.mark.parametrize("dt", [np.int32, np.float32, np.float16, np.bool_])
def test_cmp_scalar(dt):  # :44-79: scalar on the right (bool tensors against True), scalar on the left
    rng = np.random.default_rng(np.dtype(dt).itemsize)
    a = rng.integers(0, 1024, (1024, 32)).astype(dt)
    if dt in (np.float32, np.float16):
        a[0] = np.nan
    s = True if dt == np.bool_ else 30

    def g(k):
        x = k.copy(k.load(a))
        outs = [(k.store(k.copy(getattr(k, name)(x, s))), fn(a, s), 0) for name, fn in OPS]
        if dt != np.bool_:
            outs += [(k.store(k.copy(getattr(k, name)(s, x))), fn(s, a), 0) for name, fn in OPS]
        return outs
    run_graph("split", g)


def test_cmp_long_and_narrow():  # :81-95, :157-167
    rng = np.random.default_rng(3)
    a, b = rng.integers(0, 1024, (100000, 1)).astype(np.float16), rng.integers(0, 1024, (100000, 7)).astype(np.float16)
    run_graph("", lambda k: (lambda x, y: [(k.store(k.equal(x, y)), a == b, 0), (k.store(k.not_equal(x, y)), a != b, 0)])(k.load(a), k.load(b)))
    c = rng.normal(-1, 1, [2048, 9]).astype(np.float16)
    run_graph("", lambda k: [(k.store(k.cast(k.less_equal(k.cast(k.load(c), "float32"), 2.0), "bool")), c <= 2, 0)])


def test_cmp_int_full_range():  # :97-110
    rng = np.random.default_rng(4)
    a = rng.integers(-2147483648, 2147483647, (1024, 1024)).astype(np.int32)
    b = rng.integers(-2147483648, 2147483647, (1024, 1024)).astype(np.int32)
    b[::7] = a[::7]

    def g(k):
        x, y = k.load(a), k.load(b)
        return [(k.store(getattr(k, name)(x, y)), fn(a, b), 0) for name, fn in OPS]
    run_graph("split", g)


def test_cmp_of_copies():  # :113-139
    rng = np.random.default_rng(5)
    a, b = rng.integers(0, 1024, (32, 512)).astype(np.float16), rng.integers(0, 1024, (32, 512)).astype(np.float16)
    run_graph("", lambda k: [(k.store(k.equal(k.copy(k.load(a)), k.copy(k.load(b)))), a == b, 0)])
    run_graph("", lambda k: [(k.store(k.equal(k.copy(k.load(a)), 1.0)), a == 1.0, 0)])


def test_two_kernels_of_different_types_in_a_row():  # :246-258
    rng = np.random.default_rng(6)
    for dt in (np.int32, np.float16):
        data = rng.integers(0, 1024, (1024, 2000)).astype(dt)
        run_graph("", lambda k: [(k.store(k.copy(k.load(data))), data, 0)])


@pytest.mark.parametrize("shape", [(1024, 32), (13, 131), (16, 11), (3, 3)])
@pytest.mark.parametrize("dt", [np.float32, np.float16, np.int32])
def test_select(shape, dt):  # tests/ut/test_select.py:21-40
    rng = np.random.default_rng(shape[0] + np.dtype(dt).itemsize)
    a, b, c, d = (rng.integers(0, 1024, shape).astype(dt) for _ in range(4))

    def g(k):
        e, f = k.load(a), k.load(b)
        return [(k.store(k.select(k.greater(e, f), k.add(e, f), k.add(k.load(c), k.load(d)))), np.where(a > b, a + b, c + d).astype(dt), 0)]
    run_graph("", g)


def test_select_fp32_compare_result_feeds_select_directly():  # :43-61
    rng = np.random.default_rng(7)
    a, b, c, d = (rng.normal(0, 1, (128, 777)).astype(np.float32) for _ in range(4))
    t = run_graph("", lambda k: [(k.store(k.select(k.greater(k.load(a), k.load(b)), k.load(c), k.load(d))), np.where(a > b, c, d), 0)])
    assert "cast" not in t.das().lower()


@pytest.mark.parametrize("dt", [np.float32, np.float16, np.int32])
def test_select_broadcast(dt):  # :64-83
    rng = np.random.default_rng(np.dtype(dt).itemsize)
    a, b = rng.integers(0, 1024, (1, 10, 1, 1, 50)).astype(dt), rng.integers(0, 1024, (1, 1, 20, 30, 1)).astype(dt)
    c, d = rng.integers(0, 1024, (7, 1, 1, 1, 50)).astype(dt), rng.integers(0, 1024, (1, 1, 1, 30, 1)).astype(dt)

    def g(k):
        e, f = k.load(a), k.load(b)
        return [(k.store(k.select(k.greater(e, f), k.add(e, f), k.add(k.load(c), k.load(d)))), np.where(a > b, a + b, c + d).astype(dt), 0)]
    run_graph("", g)


@pytest.mark.parametrize("shape", [(1024, 32), (13, 131), (16, 11), (3, 3)])
@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_select_bool_input(shape, dt):  # :86-100
    rng = np.random.default_rng(shape[1])
    a, b, c = rng.random(shape).astype(dt), rng.random(shape).astype(dt), rng.choice([True, False], shape).astype(bool)
    run_graph("", lambda k: [(k.store(k.select(k.load(c), k.load(a), k.load(b))), np.where(c, a, b), 0)])


def test_select_scalar_operands():  # :103-114: 0-d condition and 0-d branch
    rng = np.random.default_rng(8)
    a, b = rng.integers(0, 1024, (1024, 10)).astype(np.float16), np.asarray(rng.integers(0, 1024, ())).astype(np.float16)
    for cv in (True, False):
        c = np.array(cv)
        run_graph("", lambda k: [(k.store(k.select(k.load(c), k.load(a), k.load(b))), np.where(c, a, b).astype(np.float16), 0)])
