"""GPU parity: broadcast, reduce, reshape, graph cutting and dynamic shapes (reference tests cited per case)."""
import numpy as np
import pytest

from dvm_amd import DataType
from dvm_amd.tester import Tester
from tests.util import run_parity

pytestmark = pytest.mark.gpu


def test_add_example():  # examples/01_add.py:19-34 (BASELINE config 1)
    import dvm_amd as dvm

    @dvm.kernel
    def my_add(k, x, y):
        return k.store(k.add(k.load(x, dvm.float32), k.load(y, dvm.float32)))
    x, y = np.full([32, 32], 0.1, np.float32), np.full([32, 32], 0.3, np.float32)
    assert np.array_equal(my_add(x, y), x + y)
    x, y = np.full([32, 1], 0.2, np.float32), np.full([32, 512], 0.7, np.float32)
    assert np.array_equal(my_add(x, y), x + y)  # same kernel object, new shapes


@pytest.mark.parametrize("case", [((32, 1), (32, 512)), ((1, 512), (32, 512)), ((4, 1, 7, 1), (4, 3, 7, 5)), ((1,), (33, 9)),
                                  ((2, 3, 1, 5), (2, 3, 4, 5)), ((16, 1, 131), (16, 4, 131))])
@pytest.mark.parametrize("dt", [np.float32, np.float16, np.int32, np.bool_])
def test_broadcast(case, dt):  # tests/ut/test_broadcast.py:24-165
    src, dst = case
    rng = np.random.default_rng(len(dst))
    x = (rng.normal(0, 10, src)).astype(dt)
    run_parity(lambda k, a: k.broadcast(a, list(dst)), [x], golden=np.broadcast_to(x, dst), eps=0)
    if dt not in (np.bool_,):
        y = (rng.normal(0, 10, dst)).astype(dt)
        with np.errstate(over="ignore"):
            run_parity(lambda k, a, b: k.add(a, b), [x, y], golden=x + y, eps=0 if dt == np.int32 else None)


def test_broadcast_scalar_and_bf16():  # tests/ut/test_broadcast.py:257-277
    run_parity(lambda k, a: k.add(k.full(0.3, [3, 10], "float32"), a), [np.zeros([3, 10], np.float32)], golden=np.full([3, 10], np.float32(0.3)))
    x = np.random.default_rng(2).normal(0, 1, [7, 1]).astype(np.float32)
    outs = run_parity(lambda k, a: k.broadcast(a, [7, 33]), [x], dtypes=["bfloat16"], eps=0)
    assert outs[0].shape == (7, 33)


@pytest.mark.parametrize("dim", [64, 256, 251])
def test_sum_last_axis(dim):  # tests/ut/test_reduce.py:24-33
    x = np.random.default_rng(dim).normal(-0.5, 0.5, [10, dim]).astype(np.float32)
    run_parity(lambda k, a: [k.sum(a, (1,), True), k.sum(a, (1,), False)], [x],
               golden=[np.sum(x, 1, keepdims=True), np.sum(x, 1)])


@pytest.mark.parametrize("shape", [(10, 6, 64), (10, 6, 60), (10, 2, 6128)])
def test_sum_middle_axis(shape):  # tests/ut/test_reduce.py:36-45
    x = np.random.default_rng(shape[2]).normal(-0.5, 0.5, shape).astype(np.float32)
    run_parity(lambda k, a: k.sum(a, (1,), False), [x], golden=np.sum(x, 1))


@pytest.mark.parametrize("ij", [(1, 1), (3, 5), (7, 9), (13, 11), (17, 3), (5, 31), (9, 9)])
def test_sum_023(ij):  # tests/ut/test_reduce.py:48-58
    x = np.random.default_rng(ij[0]).normal(-0.5, 0.5, [3, 1280, ij[0], ij[1]]).astype(np.float32)
    run_parity(lambda k, a: k.sum(a, (0, 2, 3), True), [x], golden=np.sum(x, (0, 2, 3), keepdims=True), eps=1e-4)


@pytest.mark.parametrize("dims", [(0,), (6,), (1, 3), (0, 2, 5), (2, 4, 6), (0, 1, 2, 3, 4, 5, 6), (1, 2), (3, 5, 6)])
def test_sum_rank7(dims):  # tests/ut/test_reduce.py:61-71
    x = np.random.default_rng(len(dims)).normal(-0.5, 0.5, [6, 4, 2, 5, 1, 3, 8]).astype(np.float32)
    run_parity(lambda k, a: [k.sum(a, dims, True), k.sum(a, dims, False)], [x],
               golden=[np.sum(x, dims, keepdims=True), np.sum(x, dims)], eps=1e-5)


@pytest.mark.parametrize("dim", [1001, 1024])
def test_sum_axis0_constant(dim):  # tests/ut/test_reduce.py:74-83
    x = np.full([64, dim], 0.01, np.float32)
    run_parity(lambda k, a: k.sum(a, (0,), False), [x], golden=np.full([dim], 0.64, np.float32))


@pytest.mark.parametrize("shape,dims", [((4096, 40000), (1,)), ((1024, 1000), (0, 1)), ((32, 2048), (1,)), ((3, 20000), (0,)),
                                        ((2048, 3201), (1,)), ((7, 5, 3), (1,)), ((128, 1), (0,)), ((1, 4096), (1,))])
def test_sum_regression_shapes(shape, dims):  # tests/ut/test_reduce.py:86-108, tests/st/test_bugfix.py:20-53,98
    x = np.random.default_rng(shape[0]).normal(-0.5, 0.5, shape).astype(np.float32)
    run_parity(lambda k, a: k.sum(a, dims, False), [x], golden=np.sum(x.astype(np.float64), dims).astype(np.float32), eps=1e-4)


@pytest.mark.parametrize("shape,dims", [((77, 513), (1,)), ((77, 513), (0,)), ((3, 1280, 7, 9), (0, 2, 3)), ((6, 4, 2, 5, 1, 3, 8), (1, 3))])
@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_max_min(shape, dims, dt):  # ops the reference's CUDA VM lacks; NumPy golden, exact (tests/ut/test_reduce.py:86-133)
    x = np.random.default_rng(shape[0]).normal(-0.5, 0.5, shape).astype(dt)
    run_parity(lambda k, a: [k.max(a, dims, True), k.min(a, dims, False)], [x],
               golden=[np.max(x, dims, keepdims=True), np.min(x, dims)], eps=0)


def test_fused_reduce_graphs():  # tests/ut/test_reduce.py:232-308
    x = np.full([32, 2048], 0.01, np.float32)
    run_parity(lambda k, a: k.sum(k.add(a, a), (1,), True), [x], golden=np.full([32, 1], 40.96, np.float32))
    y = np.random.default_rng(1).uniform(0, 1, [1024, 1000]).astype(np.float32)
    run_parity(lambda k, a: k.sum(k.copy(a), (0, 1), False), [y], golden=np.sum(y.astype(np.float64), (0, 1)).astype(np.float32), eps=1e-4)
    b = np.random.default_rng(2).normal(0, 1, [1, 64, 1, 1]).astype(np.float32)
    z = np.random.default_rng(3).normal(0, 1, [3, 64, 7, 9]).astype(np.float32)

    def g(k, p, q):
        s = k.add(k.broadcast(p, [3, 64, 7, 9]), q)
        return [k.sum(s, (0, 2, 3), True), s]
    run_parity(g, [b, z], ker="split", golden=[np.sum((b + z).astype(np.float64), (0, 2, 3), keepdims=True).astype(np.float32), b + z], eps=1e-4)


def test_reduce_then_consumers_split_graph():  # tests/ut/test_eager_fusion.py:25-212 (graph-cutting cases)
    rng = np.random.default_rng(4)
    x = rng.normal(0, 1, [64, 300]).astype(np.float32)

    def softmax(k, a):
        m = k.max(a, (1,), True)
        e = k.exp(k.sub(a, m))
        return [k.div(e, k.sum(e, (1,), True)), m]
    ex = np.exp(x - x.max(1, keepdims=True))
    run_parity(softmax, [x], ker="split", golden=[ex / ex.sum(1, keepdims=True), x.max(1, keepdims=True)], eps=1e-5)

    # a reduce result that two consumers and a store share; a dead node; a shared load
    def g(k, a):
        s = k.sum(a, (1,), True)
        _dead = k.exp(a)
        return [k.mul(a, s), k.add(s, 1.0), k.sub(a, k.mul(s, 1.0 / 300))]
    s = x.astype(np.float64).sum(1, keepdims=True).astype(np.float32)
    run_parity(g, [x], ker="split", golden=[x * s, s + 1, x - s * np.float32(1.0 / 300)], eps=1e-4)

    # reduces over different axes of one input cannot share a kernel: the graph is cut, results still right
    def g2(k, a):
        return [k.sum(a, (0,), True), k.sum(a, (1,), True), k.add(k.sum(a, (1,), True), k.sum(k.mul(a, a), (1,), True))]
    run_parity(g2, [x], ker="split", eps=1e-4,
               golden=[x.astype(np.float64).sum(0, keepdims=True), x.astype(np.float64).sum(1, keepdims=True),
                       (x.astype(np.float64).sum(1, keepdims=True) + (x.astype(np.float64) ** 2).sum(1, keepdims=True))])


def test_reshape_graphs():  # tests/ut/test_reshape.py:24-160
    for dims in [(2,), (1,)]:
        b = np.full((10, 3, 1), 0.1, np.float32)
        run_parity(lambda k, a: k.sum(k.reshape(k.broadcast(a, [10, 3, 4]), [1, 10, 12]), dims, True), [b], ker="split",
                   golden=np.sum(np.broadcast_to(b, (10, 3, 4)).reshape(1, 10, 12), dims, keepdims=True))
    x = np.full((16, 16), 81.0, np.float32)
    run_parity(lambda k, a: k.sqrt(k.reshape(k.sqrt(a), [32, 8])), [x], ker="split", golden=np.full((32, 8), 3.0, np.float32))
    run_parity(lambda k, a: k.cast(k.sqrt(k.reshape(k.sqrt(a), [32, 8])), "float16"), [x], ker="split", golden=np.full((32, 8), 3.0, np.float16))
    rng = np.random.default_rng(5)
    c, p, q = rng.choice([True, False], (3, 3)), np.full((9,), 1.0, np.float32), np.full((3, 3), 2.0, np.float32)
    run_parity(lambda k, cc, pp, qq: k.select(cc, k.reshape(pp, [3, 3]), qq), [c, p, q], ker="split", golden=np.where(c, p.reshape(3, 3), q))
    y = np.full([1, 8], 0.3, np.float32)
    run_parity(lambda k, a: k.broadcast(k.reshape(k.broadcast(a, [10, 8]), [10, 1, 8]), [10, 4, 8]), [y], ker="split", golden=np.full([10, 4, 8], np.float32(0.3)))
    z = np.full([10, 3, 4], 0.3, np.float32)
    run_parity(lambda k, a: k.broadcast(k.reshape(a, [1, 10, 12]), [8, 10, 12]), [z], ker="split", golden=np.full([8, 10, 12], np.float32(0.3)))
    a = rng.uniform(0.1, 1, (54, 89)).astype(np.float32)
    run_parity(lambda k, v: k.add(k.sqrt(k.reshape(v, [89, 54])), k.reshape(k.reciprocal(v), [89, 54])), [a], ker="split",
               golden=(np.sqrt(a) + np.reciprocal(a)).reshape(89, 54))


@pytest.mark.parametrize("shape", [(13, 131), (128, 7), (5, 1023), (1, 1), (2, 3, 5, 7)])
@pytest.mark.parametrize("dt", [np.float32, np.float16, np.int32, np.bool_])
def test_unaligned_shapes(shape, dt):  # tests/ut/test_unalign.py:25-72, tests/ut/test_misc.py:26
    rng = np.random.default_rng(shape[-1])
    x = rng.normal(0, 10, shape).astype(dt)
    y = rng.normal(0, 10, shape).astype(dt)
    if dt == np.bool_:
        run_parity(lambda k, a, b: [k.copy(a), k.logical_or(a, b)], [x, y], golden=[x, np.logical_or(x, y)])
    else:
        with np.errstate(over="ignore"):
            run_parity(lambda k, a, b: [k.copy(a), k.mul(a, b)], [x, y], golden=[x, x * y], eps=0 if dt == np.int32 else None)


def _dyn_sum_kernel():
    t = Tester("vector:dyn")
    x = t.load([1, 1, 4096], "float16")
    y = t.load([1, 1, 4096], "float16")
    s = t.add(x, y)
    f = t.cast(s, "float32")
    outs = [t.store(s), t.store(f), t.store(t.sum(t.mul(f, f), (2,), True))]
    return t, (x, y), outs


def test_dynamic_shapes():  # tests/ut/test_dynamic_shape.py:68-114,137-162 (closest reference test to BASELINE config 3)
    t, (x, y), outs = _dyn_sum_kernel()
    for rows in (2685, 2686, 2687, 1, 64):
        np.random.seed(rows)
        a = Tester.fast_random_normal(0, 1, [1, rows, 4096]).astype(np.float16)
        b = Tester.fast_random_normal(0, 1, [1, rows, 4096]).astype(np.float16)
        t.input(x, a)
        t.input(y, b)
        t.run()
        s = a + b
        assert np.array_equal(t.output(outs[0]), s)
        assert np.array_equal(t.output(outs[1]), s.astype(np.float32))
        want = np.sum(s.astype(np.float64) ** 2, 2, keepdims=True)
        assert np.allclose(t.output(outs[2]), want, rtol=1e-4, atol=1e-4)


def test_scalar_ref_updates():  # tests/ut/test_elemwise.py:500-532
    t = Tester("vector:dyn")
    x = t.load([1024], "float32")
    sf = t.scalar()
    si = t.scalar(DataType.int32)
    xi = t.load([1024], "int32")
    o1 = t.store(t.mul(x, sf))
    o2 = t.store(t.add(xi, si))
    a = np.random.default_rng(0).normal(-10, 10, [1024]).astype(np.float32)
    ai = np.random.default_rng(1).integers(-100, 100, [1024]).astype(np.int32)
    for fv, iv in [(0.5, 3), (-2.25, -7), (10.0, 11111)]:
        t.input(x, a)
        t.input(xi, ai)
        sf.update(fv)
        si.update(iv)
        t.run()
        assert np.array_equal(t.output(o1), a * np.float32(fv))
        assert np.array_equal(t.output(o2), ai + np.int32(iv))


def test_zero_size():  # tests/ut/test_codegen.py:116-164
    t = Tester("vector")
    x = t.load(np.zeros([0, 16], np.float32))
    s = t.store(t.sum(x, (0,), False))
    e = t.store(t.add(x, 1.0))
    t.run()
    assert np.array_equal(t.output(s), np.zeros([16], np.float32))
    assert t.output(e).shape == (0, 16)


def test_wide_build_matches(monkeypatch):
    # the optional four-slabs-per-lane build of the VM (DVM_VEC_WIDE=1) computes the same results
    monkeypatch.setenv("DVM_VEC_WIDE", "1")
    rng = np.random.default_rng(77)
    x = rng.normal(0, 1, [6, 5, 700]).astype(np.float32)
    g = rng.normal(0, 1, [5, 1]).astype(np.float32)

    def build(k, a, b):
        m = k.mul(k.sum(a, (0, 2), True), 1.0 / 4200)
        d = k.sub(a, m)
        return [k.mul(d, b), k.max(a, (2,), False), k.add(a, 1.0)]
    outs = run_parity(build, [x, g], golden=[(x - x.mean((0, 2), keepdims=True)) * g, x.max(2), x + 1], eps=1e-5)
    assert outs[0].shape == x.shape
    t = Tester("split", run_mode="das")
    t.store(t.sum(t.load(x), (2,), False))
    t.codegen()
    assert " wide " in t.das()


@pytest.mark.parametrize("shape,axis", [((33, 100), 0), ((70, 257), 0), ((5, 3000), 1), ((3, 5000, 8), 1)])
def test_reduce_result_outlives_temporaries_of_later_rounds(shape, axis):
    # a second sweep of several rounds reads the reduce result in every round: temporaries of the first round
    # must not take its register (two outputs with a compare each make the emitter park a mask per output)
    x = np.random.default_rng(1161).uniform(0.25, 2.0, shape).astype(np.float32)

    def build(k, a):
        m = k.max(a, (axis,), True)
        m2 = k.add(m, m)
        first = k.select(k.greater(a, m2), a, m2)
        second = k.select(k.greater(m, a), m, a)
        return [first, k.sub(second, a)]
    mx = x.max(axis, keepdims=True)
    run_parity(build, [x], golden=[np.broadcast_to(2 * mx, shape), np.broadcast_to(mx, shape) - x], eps=0)


@pytest.mark.parametrize("three", [False, True])
def test_copy_beside_a_reduce_to_one_element(three):
    # an output of one element relates to no other output; the copies next to it are matched through the
    # reduce's input, which has the dims the launch walks
    x = np.random.default_rng(18).uniform(0.25, 2.0, [1, 2, 3000]).astype(np.float16)

    def build(k, a):
        f = k.cast(a, "float32")
        flat = k.reshape(f, [6000])
        other = k.reshape(k.mul(f, f), [6000])
        outs = [other, k.sum(flat, (0,), True)]
        return outs + [k.add(flat, 0.0)] if three else outs
    xf = x.astype(np.float32).reshape(6000)
    golden = [xf * xf, xf.sum(keepdims=True)] + ([xf] if three else [])
    run_parity(build, [x], golden=golden, eps=1e-5)


def test_operators_on_a_value_of_rank_zero():  # src/ops.cc:3080-3117: a reduce over every dim without keepdims
    x = np.random.default_rng(5).uniform(-2, 2, [257]).astype(np.float32)

    def build(k, a):
        m = k.min(a, (0,), False)
        r = k.floor(k.add(m, 0.25))
        return [m, r, k.mul(a, r)]
    outs = run_parity(build, [x], golden=[x.min(), np.floor(x.min() + np.float32(0.25)), x * np.floor(x.min() + np.float32(0.25))], eps=0)
    assert outs[0].shape == () and outs[1].shape == () and outs[2].shape == (257,)
    bf = Tester.convert_from_bf16(Tester.convert_to_bf16(np.float32(1.5)))
    assert bf.shape == () and float(bf) == 1.5


@pytest.mark.parametrize("n,hint", [(256 * 50 + 100, (0, 0, 51, 256)), (249 * 50 + 223, (0, 0, 51, 249)), (501 * 20, (0, 0, 20, 501))])
def test_sum_of_a_long_vector_with_a_tiling_hint(n, hint):  # tests/ut/test_reduce.py:310-325 (the hint fixes the reference's tiles)
    a = np.random.default_rng(n).standard_normal([n], dtype=np.float32)
    t = Tester()
    t.store_expect(t.sum(t.load(a), (0,), True), np.sum(a.astype(np.float64), axis=(0,), keepdims=True), 1e-4)
    t.tile(*hint)
    assert t.run_check()


def test_sum_over_both_axes_of_rows_of_two():  # tests/ut/test_reduce.py:328-338
    rng = np.random.default_rng(8002)
    a0, a1 = rng.standard_normal([8002, 2], dtype=np.float32), rng.standard_normal([8002, 1], dtype=np.float32)
    t = Tester()
    t.store_expect(t.sum(t.add(t.load(a0), t.load(a1)), [0, 1], False), np.sum((a0 + a1).astype(np.float64), axis=(0, 1)), 1e-4)
    t.tile(1, 1, 8)
    assert t.run_check()


def test_sum_of_a_broadcast_stored_beside_its_input():  # tests/ut/test_reduce.py:296-307
    a = (np.random.default_rng(12).standard_normal([32, 12, 1, 1]) * 0.5 - 0.5).astype(np.float32)
    wide = np.broadcast_to(a, [32, 12, 111, 111]) + np.float32(0.1)
    t = Tester()
    x = t.add(t.broadcast(t.load(a), [32, 12, 111, 111]), 0.1)
    t.store_expect(t.sum(x, [0, 2, 3], False), np.sum(wide.astype(np.float64), axis=(0, 2, 3)), 1e-4)
    t.store_expect(x, wide)
    assert t.run_check()


def test_tensors_beyond_four_gigabytes():
    # byte offsets past 2^32 in each schedule: row sums and a normalise sweep (reduce over the innermost axis), column sums
    # (the innermost axis kept, shared between workgroups), a matmul operand; expectations in closed form
    rows, cols = 40960, 32768
    x = np.empty([rows, cols], np.float32)
    x[:] = (np.arange(rows) % 13).astype(np.float32)[:, None]
    x[:, ::2] *= -0.5
    row_sum = ((np.arange(rows) % 13).astype(np.float64) * (cols / 2) * 0.5)[:, None]
    t = Tester("split")
    st = t.store(t.sum(t.load(x), (1,), True))
    t.run()
    assert np.allclose(t.output(st), row_sum, rtol=1e-5)
    t = Tester("split")
    xl = t.load(x)
    st = t.store(t.sub(xl, t.mul(t.sum(xl, (1,), True), 1.0 / cols)))
    t.run()
    assert np.allclose(t.output(st), x - (row_sum / cols).astype(np.float32), rtol=1e-5, atol=1e-4)
    tall = x.reshape(rows * 2, cols // 2)
    t = Tester("split")
    st = t.store(t.sum(t.load(tall), (0,), True))
    t.run()
    assert np.allclose(t.output(st), tall.astype(np.float64).sum(0, keepdims=True), rtol=1e-4)
    del x, tall
    m, k, n = 65536, 40960, 128
    a = np.empty([m, k], np.float16)
    a[:] = (np.arange(m) % 7).astype(np.float16)[:, None]
    t = Tester("mix")
    st = t.store(t.matmul(t.load(a), t.load(np.full([k, n], 0.125, np.float16)), False, False))
    t.run()
    want = ((np.arange(m) % 7) * k * 0.125).astype(np.float32)[:, None] * np.ones([1, n], np.float32)
    assert np.array_equal(t.output(st).astype(np.float32), want)


@pytest.mark.parametrize("rows,cols", [(7, 8), (300, 4096), (33, 1000)])
@pytest.mark.parametrize("red", ["min", "max", "sum"])
def test_reduce_over_the_repeats_of_a_broadcast_that_is_used_again(rows, cols, red):
    # The value that is reduced over axis 0 does not vary along it (a row repeated): what follows takes it from the
    # accumulator of the last round instead of loading it again, so the load of that sweep must leave it there.
    # (The load that fetches several rounds per trip and reduces them itself did not.)
    x = np.random.default_rng(rows).uniform(0.25, 2.0, [1, cols]).astype(np.float32)
    want = {"min": x, "max": x, "sum": x * np.float32(rows)}[red] + np.broadcast_to(x, (rows, cols))

    def g(k, a):
        b = k.broadcast(a, [rows, cols])
        m = getattr(k, red)(b, (0,), True)
        picked = k.select(k.greater(m, a), a, m)  # (the reduce result either way for min; keeps the graph of the failing case)
        return k.add(picked if red == "min" else m, b)
    run_parity(g, [x], ker="split", golden=want, eps=1e-5)
