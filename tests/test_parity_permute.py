"""GPU parity: views of computed values, restating tests/ut/test_permute.py of the reference and the Slice / Split
cases of tests/ut/test_view_sch.py and tests/ut/test_spec_vector.py (cited per test): Permute, Slice (box and
single-dim form), Split. Same shapes and NumPy expectations as there, default kernel type; every graph also
runs on the CPU oracle. Here these operators are views: their input stays (or is written) in memory once and the
consumers read it through strides, so what the graphs probe is which launch writes and which reads, through what
strides and offset."""
import numpy as np
import pytest

from dvm_amd._core import DataType
from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def rng(seed=0):
    return np.random.default_rng(seed)


def dense(shape):
    st = [1] * len(shape)
    for i in range(len(shape) - 1, 0, -1):
        st[i - 1] = st[i] * shape[i]
    return st


# ---- Permute, tests/ut/test_permute.py ----

def test_permute_from_load():  # :36-43
    a = rng(1).normal(-0.5, 0.5, [10, 20, 32]).astype(np.float16)
    run_graph("", lambda k: [(k.store(k.permute(k.load(a), [1, 0, 2])), np.transpose(a, (1, 0, 2)), 0)])


@pytest.mark.parametrize("in_shape, b_shape, perm", [([10, 1, 200], [10, 20, 200], [1, 0, 2]), ([10, 1, 1, 200], [10, 20, 5, 200], [0, 2, 1, 3]),
                                                     ([10, 1, 1, 200], [10, 20, 5, 200], [2, 1, 0, 3]), ([1, 1, 10, 200], [10, 20, 10, 200], [3, 1, 2, 0])])
def test_permute_broadcast(in_shape, b_shape, perm):  # :46-60
    a = rng(2).normal(0, 0.5, in_shape).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.permute(k.broadcast(k.view_load(in_shape, dense(in_shape), a), b_shape), perm)),
                              np.transpose(np.broadcast_to(a, b_shape), perm), 0)])


@pytest.mark.parametrize("in_shape, dims, perm", [([10, 20, 512], (1,), [1, 0, 2]), ([10, 2, 40, 600], (0, 3), [1, 0, 2, 3]),
                                                  ([10, 2, 40, 600], (0, 3), [2, 1, 0, 3]), ([10, 20, 512], (1, 2), [1, 0, 2])])
def test_permute_reduce(in_shape, dims, perm):  # :63-78 (the reference's 6000-wide rows at 600)
    a = rng(3).normal(-0.3, 0.5, in_shape).astype(np.float32)
    g = np.transpose(np.sum(a, dims, keepdims=True) + np.float32(0.1), perm)
    run_graph("", lambda k: [(k.store(k.permute(k.add(k.sum(k.view_load(in_shape, dense(in_shape), a), dims, True), 0.1), perm)), g, 1e-4)], oracle_eps=1e-4)


def test_permute_backward():  # :81-92 (broadcast after the permute, stored through strides)
    a = rng(4).normal(-0.3, 0.5, [20, 1, 200]).astype(np.float32)
    e = (np.broadcast_to(np.transpose(a + np.float32(0.1), [2, 1, 0]), [200, 30, 20]) * np.float32(0.5)).astype(np.float32)

    def g(k):
        x4 = k.mul(k.broadcast(k.permute(k.add(k.load(a), 0.1), [2, 1, 0]), [200, 30, 20]), 0.5)
        return [(k.view_store_expect(x4, dense([200, 30, 20]), e), e, None)]
    run_graph("", g)


def test_permute_nest():  # :95-104
    a = rng(5).normal(0.0, 0.5, [10, 20, 1]).astype(np.float16)
    g = np.transpose(np.broadcast_to(np.transpose(a, (1, 0, 2)), [20, 10, 100]), (0, 2, 1))
    run_graph("", lambda k: [(k.store(k.permute(k.broadcast(k.permute(k.load(a), [1, 0, 2]), [20, 10, 100]), [0, 2, 1])), g, 0)])


def test_permute_copy_reshape():  # :107-118
    a = rng(6).normal(0.0, 0.5, [32, 1024]).astype(np.float32)
    b = rng(7).normal(0.0, 0.5, [1024, 1, 16]).astype(np.float32)
    g = np.reshape(np.transpose(a, [1, 0]), [1024, 32, 1]) + b
    run_graph("", lambda k: [(k.store(k.add(k.reshape(k.copy(k.permute(k.load(a), [1, 0])), [1024, 32, 1]), k.load(b))), g, None)])


def test_permute_chained():  # :121-128 (the reference's [50, 300, 1024] at [50, 30, 1024])
    a = rng(8).normal(0.0, 0.5, [50, 30, 1024]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.permute(k.permute(k.add(k.load(a), 0.02), [1, 0, 2]), [0, 2, 1])),
                              np.transpose(a + np.float32(0.02), (1, 2, 0)), None)])


def test_permute_side_connect():  # :131-139 (the value and its permutation meet again)
    a = rng(9).normal(0.0, 0.5, [50, 1, 1024]).astype(np.float32)

    def g(k):
        x1 = k.add(k.load(a), 0.02)
        return [(k.store(k.add(x1, k.permute(x1, [1, 0, 2]))), a + np.float32(0.02) + np.transpose(a + np.float32(0.02), (1, 0, 2)), None)]
    run_graph("", g)


def test_reshape_of_a_permuted_value_needs_a_copy():
    t = Tester("vector", run_mode="das")
    t.store(t.reshape(t.permute(t.load(np.zeros([4, 8], np.float32)), [1, 0]), [32]))
    with pytest.raises(RuntimeError, match="needs a Copy"):
        t.codegen()


# ---- Slice, tests/ut/test_spec_vector.py and tests/ut/test_view_sch.py ----

@pytest.mark.parametrize("is_split", [True, False])
def test_spec_slice(is_split):  # tests/ut/test_spec_vector.py:411-422
    a0 = rng(10).normal(0, 1, [1024, 500]).astype(np.float32)
    e = (a0 * np.float32(0.1) if is_split else a0)[100:700, 100:400] + np.float32(0.2)

    def g(k):
        x0 = k.load(a0)
        if is_split:
            x0 = k.mul(x0, 0.1)
        return [(k.store(k.add(k.slice(x0, [100, 100], [600, 300]), 0.2)), e, None)]
    run_graph("", g)


@pytest.mark.parametrize("is_split, end", [(True, 700), (True, -2), (False, 100000)])
def test_spec_slice_dim(is_split, end):  # :425-438 (begin through an updatable scalar)
    a0 = rng(11).normal(0, 1, [1024, 500]).astype(np.float32)
    src = a0 * np.float32(0.1) if is_split else a0
    t = Tester("split:dyn")
    x0 = t.load([-1, 500], "float32")
    t.input(x0, a0)
    if is_split:
        x0 = t.mul(x0, 0.1)
    b_ref = t.scalar(DataType.int32)
    b_ref.update(100)
    out = t.store(t.add(t.slice_dim(x0, 0, b_ref, end), 0.2))
    t.run()
    assert np.allclose(t.output(out), src[100:end, :] + np.float32(0.2), rtol=1e-5, atol=1e-5)
    b_ref.update(37)  # the bound is read again at the next code generation
    t.run()
    got = t.output(out)
    assert got.shape == src[37:end, :].shape and np.allclose(got, src[37:end, :] + np.float32(0.2), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape1, shape2, start, slice1, slice2", [([100, 2000], [1, 2000], [10, 30], [60, 1500], [60, 1500]),
                                                                   ([100, 2000], [100, 2000], [10, 30], [60, 1500], [60, 1]),
                                                                   ([100, 1000], [100, 1000], [0, 20], [100, 500], [100, 500])])
def test_sch_slice(shape1, shape2, start, slice1, slice2):  # tests/ut/test_view_sch.py:474-490
    a, b, c = (rng(s).normal(0, 1, sh).astype(np.float32) for s, sh in ((12, shape1), (13, shape2), (14, slice2)))
    e = (a * b)[start[0]:start[0] + slice1[0], start[1]:start[1] + slice1[1]] + c
    run_graph("", lambda k: [(k.store(k.add(k.slice(k.mul(k.load(a), k.load(b)), start, slice1), k.load(c))), e, None)])


def test_sch_slice_store():  # :493-508 (the sliced value is also stored whole)
    a = rng(15).normal(0, 1, [10, 1024]).astype(np.float32)
    x1_e = a * np.float32(0.6)
    x3_e = x1_e[2:10, :512] + np.float32(0.1)

    def g(k):
        x1 = k.mul(k.load(a), 0.6)
        x3 = k.add(k.slice(x1, [2, 0], [8, 512]), 0.1)
        return [(k.store(x1), x1_e, None), (k.store(x3), x3_e, None), (k.store(k.mul(x3, 0.4)), x3_e * np.float32(0.4), None)]
    run_graph("", g)


def test_sch_slice_broadcast():  # :511-524 (a one-column slice broadcast along the rows of another operand)
    a0 = rng(16).normal(0, 1, [10, 20]).astype(np.float32)
    a1 = rng(17).normal(0, 1, [6, 20]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.exp(k.add(k.slice(k.mul(k.load(a0), 0.1), [2, 5], [6, 1]), k.load(a1)))),
                              np.exp(a0[2:8, 5:6] * np.float32(0.1) + a1), None)])


def test_sch_slice_slice_chain():  # :527-541
    a = rng(18).normal(0, 1, [1024, 500]).astype(np.float32)
    b = rng(19).normal(0, 1, [600, 300]).astype(np.float32)
    e2 = (a + np.float32(0.1))[100:700, 100:400]

    def g(k):
        x2 = k.slice(k.add(k.load(a), 0.1), [100, 100], [600, 300])
        x5 = k.exp(k.slice(k.add(x2, k.load(b)), [50, 0], [200, 160]))
        return [(k.store(x2), e2, None), (k.store(x5), np.exp((e2 + b)[50:250, :160]), None)]
    run_graph("", g)


def test_sch_slice_slice_v_branch():  # :544-558
    a0 = rng(20).normal(0, 1, [1024, 500]).astype(np.float32)
    a1 = rng(21).normal(0, 1, [1024, 500]).astype(np.float32)
    e = a0[100:300, 100:200] * np.float32(0.1) + a1[200:400, 200:300] * np.float32(0.1)
    run_graph("", lambda k: [(k.store(k.add(k.slice(k.mul(k.load(a0), 0.1), [100, 100], [200, 100]),
                                            k.slice(k.mul(k.load(a1), 0.1), [200, 200], [200, 100]))), e, None)])


def test_sch_slice_reshape_slice_chain():  # :561-576
    a = rng(22).normal(0, 1, [1024, 500]).astype(np.float32)
    e2 = (a + np.float32(0.1))[100:700, 100:400]

    def g(k):
        x2 = k.slice(k.add(k.load(a), 0.1), [100, 100], [600, 300])
        x3 = k.reshape(k.mul(x2, 0.9), [200, 3, 300])
        x5 = k.exp(k.slice(x3, [0, 1, 0], [200, 2, 300]))
        return [(k.store(x2), e2, None), (k.store(x5), np.exp((e2 * np.float32(0.9)).reshape(200, 3, 300)[:, 1:, :]), None)]
    run_graph("", g)


def test_sch_slice_split_slice():  # :654-666
    a0 = rng(23).normal(0, 1, [500, 512]).astype(np.float32)
    e3, e4 = np.split((a0 + np.float32(0.1))[50:450, :], 2)

    def g(k):
        x2 = k.slice_dim(k.add(k.load(a0), 0.1), 0, 50, 450)
        x3, x4 = k.split(x2, 0, 200, 2)
        return [(k.store(k.exp(x3)), np.exp(e3), None), (k.store(k.slice_dim(x4, 1, 100, 300)), e4[:, 100:300], None)]
    run_graph("", g)


def test_sch_slices_of_one_value_meet_again():  # :669-694
    a0 = rng(24).normal(0, 1, [4, 600]).astype(np.float32)
    e = a0 + np.float32(0.1)

    def g1(k):
        x0 = k.add(k.load(a0), 0.1)
        return [(k.store(k.add(k.slice(x0, [0, 0], [4, 300]), k.slice(x0, [0, 150], [4, 300]))), e[:, 0:300] + e[:, 150:450], None)]

    def g2(k):
        x0 = k.add(k.load(a0), 0.1)
        p0, p1 = k.mul(k.slice(x0, [0, 0], [4, 300]), 0.5), k.add(k.slice(x0, [0, 150], [4, 300]), 0.2)
        return [(k.store(k.add(p0, p1)), e[:, 0:300] * np.float32(0.5) + (e[:, 150:450] + np.float32(0.2)), None)]
    run_graph("", g1)
    run_graph("", g2)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("shape, split_size, dim, view", [([3, 900], 300, 1, False), ([3, 500, 32], 200, 1, True)])
def test_sch_split(dtype, shape, split_size, dim, view):  # :196-217 (the last chunk is smaller)
    split_num = (shape[dim] + split_size - 1) // split_size
    a = rng(25).normal(0, 1, shape).astype(dtype)
    expects = np.split(a * dtype(0.7), [split_size * (i + 1) for i in range(split_num - 1)], dim)

    def g(k):
        x0 = k.view_load(shape, dense(shape), a) if view else k.load(a)
        parts = k.split(k.mul(x0, 0.7), dim, split_size, split_num)
        return [(k.store(k.add(s, 0.1 * (i + 1))), expects[i] + dtype(0.1 * (i + 1)), 2e-3 if dtype == np.float16 else None) for i, s in enumerate(parts)]
    run_graph("", g)


def test_split_mul_broadcast():  # :276-286 (chunks of a load: no launch writes anything twice)
    a = rng(26).normal(0, 1, [3, 900]).astype(np.float32)
    s = rng(27).normal(0, 1, [3, 1]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.mul(k.add(x, k.load(s)), 0.5)), (np.split(a, [300, 600], 1)[i] + s) * np.float32(0.5), None)
                             for i, x in enumerate(k.split(k.load(a), 1, 300, 3))])


def test_split_tree_multi_branch():  # :289-311
    a = rng(28).normal(0, 1, [6, 300]).astype(np.float32)
    c = rng(29).normal(0, 1, [2, 300]).astype(np.float32)
    d = rng(30).normal(0, 1, [2, 300]).astype(np.float32)
    sp = np.split(a, 3, 0)

    def g(k):
        xa, xc, xd = k.load(a), k.load(c), k.load(d)
        a1, a2, a3 = k.split(xa, 0, 2, 3)
        b3 = k.add(a3, xd)
        return [(k.store(k.add(xa, 0.8)), a + np.float32(0.8), None), (k.store(k.add(a1, xc)), sp[0] + c, None),
                (k.store(k.add(a2, xc)), sp[1] + c, None), (k.store(b3), sp[2] + d, None), (k.store(k.mul(b3, 0.6)), (sp[2] + d) * np.float32(0.6), None)]
    run_graph("", g)


@pytest.mark.parametrize("shape1, shape2, reshape, split_dim", [([20, 512], [20, 512], [20, 2, 256], 1), ([1, 512], [20, 512], [20 * 512], 0)])
def test_sch_split_reshape(shape1, shape2, reshape, split_dim):  # :436-452 (shapes in the style of its list)
    a, b = rng(31).normal(0, 1, shape1).astype(np.float32), rng(32).normal(0, 1, shape2).astype(np.float32)
    expect = np.split((a + b).reshape(reshape) + np.float32(0.1), 2, split_dim)

    def g(k):
        x3, x4 = k.split(k.add(k.reshape(k.add(k.load(a), k.load(b)), reshape), 0.1), split_dim, reshape[split_dim] // 2, 2)
        return [(k.store(x3), expect[0], None), (k.store(x4), expect[1], None)]
    run_graph("", g)


def test_sch_diamond_view_load():  # :764-786 (split and slice of one value; of a strided load with gaps)
    a0 = np.arange(144, dtype=np.float32).reshape(4, 36)

    def g1(k):
        x = k.add(k.view_load([4, 36], [36, 1], a0), 0.0)
        parts = k.split(x, 1, 12, 3)
        return [(k.store(k.add(parts[1], k.slice(x, [0, 12], [4, 12]))), 2 * a0[:, 12:24], 0)]
    run_graph("", g1)
    a1 = np.arange(64, dtype=np.float32).reshape(8, 8)

    def g2(k):
        vl = k.view_load([8, 4], [8, 2], a1)
        parts = k.split(vl, 1, 2, 2)
        return [(k.store(k.add(parts[1], k.slice(vl, [0, 2], [8, 2]))), 2 * a1[:, [4, 6]], 0)]
    run_graph("", g2)


def test_sch_diamond_dyn():  # :789-803 (the sliced rows stay while the input grows)
    t = Tester("vector:dyn")
    x = t.load([-1, 120], "float32")
    y = t.add(x, 0.0)
    out = t.store(t.add(t.slice(y, [0, 0], [4, 60]), t.slice(y, [0, 60], [4, 60])))
    for nrows in [4, 8, 16]:
        a = np.arange(nrows * 120, dtype=np.float32).reshape(nrows, 120)
        t.input(x, a)
        t.run()
        assert np.array_equal(t.output(out), a[:4, 0:60] + a[:4, 60:120])


# ---- Concat, tests/ut/test_view_sch.py ----

@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("shape1, shape2, shape3, shape4, axis, view", [
    ([3, 400], [3, 600], [3, 200], [3, 1200], 1, False), ([3, 400, 32], [3, 600, 32], [3, 200, 32], [3, 1, 32], 1, True),
    ([10, 400], [20, 400], [30, 400], [60, 1], 0, False)])
def test_sch_concat(dtype, shape1, shape2, shape3, shape4, axis, view):  # :109-137
    a0, a1, a2, a3 = (rng(40 + i).normal(0, 1, sh).astype(dtype) for i, sh in enumerate((shape1, shape2, shape3, shape4)))
    expect = np.concatenate([a0 + dtype(0.1), a1 * dtype(0.6), a2], axis=axis) + a3
    eps = 2e-3 if dtype == np.float16 else None

    def g(k):
        x5 = k.concat([k.add(k.load(a0), 0.1), k.mul(k.load(a1), 0.6), k.load(a2)], axis)
        if view:
            return [(k.view_store_expect(k.add(x5, k.view_load(shape4, dense(shape4), a3)), dense(expect.shape), expect), expect, eps)]
        return [(k.store(k.add(x5, k.load(a3))), expect, eps)]
    run_graph("", g)


def test_sch_concat_many_parts():  # :140-160 (one large part and 69 tiny ones; the reference's 137862 rows at 13786)
    r = rng(44)
    arrs = [r.normal(0, 1, [13786, 32]).astype(np.float32)] + [r.normal(0, 1, [2, 32]).astype(np.float32) for _ in range(69)]
    expect = np.concatenate([a + np.float32(0.1) for a in arrs], axis=0) * np.float32(0.5)
    run_graph("", lambda k: [(k.store(k.mul(k.concat([k.add(k.load(a), 0.1) for a in arrs], 0), 0.5)), expect, None)])


def test_sch_concat_dyn():  # :163-193 (shapes and ranks change between runs)
    t = Tester("vector:dyn")
    x0, x1, x4 = t.load([-1], "float32"), t.load([-1], "float32"), t.load([-1], "float32")
    out = t.store(t.add(t.concat([t.add(x0, 0.1), t.mul(x1, 0.6), x4], 1), 0.2))
    r = rng(45)
    for s1, s2, s3 in [([3, 300], [3, 400], [3, 200]), ([3, 300, 16], [3, 400, 16], [3, 200, 16]), ([10, 1000], [10, 800], [10, 200])]:
        a0, a1, a2 = (r.normal(0, 1, s).astype(np.float32) for s in (s1, s2, s3))
        t.input(x0, a0)
        t.input(x1, a1)
        t.input(x4, a2)
        t.run()
        expect = np.concatenate([a0 + np.float32(0.1), a1 * np.float32(0.6), a2], axis=1) + np.float32(0.2)
        got = t.output(out)
        assert got.shape == expect.shape and np.allclose(got, expect, rtol=1e-5, atol=1e-5)


def test_concat_add_broadcast():  # :261-272
    a, b, s = (rng(46 + i).normal(0, 1, sh).astype(np.float32) for i, sh in enumerate(([3, 300], [3, 400], [3, 1])))
    run_graph("", lambda k: [(k.store(k.add(k.concat([k.load(a), k.load(b)], 1), k.load(s))), np.concatenate([a, b], axis=1) + s, None)])


def test_concat_one_row_after_many():  # :316-327 (no part is dropped, however small its share)
    lhs, rhs = rng(49).normal(0, 1, [24576, 32]).astype(np.float32), rng(50).normal(0, 1, [1, 32]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.concat([k.load(lhs), k.load(rhs)], 0)), np.concatenate([lhs, rhs], axis=0), 0)])


def test_sch_concat_shared_load():  # :330-340 (one load is two of the parts)
    a0, a1 = rng(51).normal(0, 1, [3, 400]).astype(np.float16), rng(52).normal(0, 1, [3, 600]).astype(np.float16)

    def g(k):
        x0 = k.load(a0)
        return [(k.store(k.add(k.concat([x0, x0, k.load(a1)], 1), 0.1)), np.concatenate([a0, a0, a1], axis=1) + np.float16(0.1), 2e-3)]
    run_graph("", g)


def test_sch_concat_part_also_stored():  # :343-356
    a0, a1 = rng(53).normal(0, 1, [3, 400]).astype(np.float16), rng(54).normal(0, 1, [3, 600]).astype(np.float16)
    e0 = a0 * np.float16(0.5)

    def g(k):
        x0 = k.mul(k.load(a0), 0.5)
        x3 = k.add(k.concat([x0, k.load(a1)], 1), 0.1)
        return [(k.store(x0), e0, 2e-3), (k.store(x3), np.concatenate([e0, a1], axis=1) + np.float16(0.1), 2e-3)]
    run_graph("", g)


def test_sch_split_and_concat_with_stores_on_the_side():  # :359-402
    a0, a1, a5 = (rng(55 + i).normal(0, 1, sh).astype(np.float16) for i, sh in enumerate(([3, 400], [3, 1], [3, 400])))
    ay = rng(58).normal(0, 1, [3, 200]).astype(np.float16)
    ay2 = rng(59).normal(0, 1, [3, 800]).astype(np.float16)
    a1w = rng(60).normal(0, 1, [3, 400]).astype(np.float16)

    def g_split(k):
        x1 = k.load(a1)
        x2 = k.add(k.load(a0), x1)
        x6 = k.sub(k.load(a5), x1)
        s0, s1 = k.split(x2, 1, 200, 2)
        sp = np.split(a0 + a1, [200], 1)
        return [(k.store(x2), a0 + a1, 2e-3), (k.store(x6), a5 - a1, 2e-3), (k.store(k.add(s0, k.load(ay))), sp[0] + ay, 2e-3), (k.store(s1), sp[1], 2e-3)]

    def g_concat(k):
        x1 = k.load(a1w)
        x2 = k.add(k.load(a0), x1)
        x6 = k.sub(k.load(a5), x1)
        y2 = k.add(k.load(ay2), k.concat([x2, x6], 1))
        return [(k.store(x2), a0 + a1w, 2e-3), (k.store(y2), np.concatenate([a0 + a1w, a5 - a1w], axis=1) + ay2, 4e-3)]
    run_graph("", g_split)
    run_graph("", g_concat)


@pytest.mark.parametrize("in_shape, cat_dim, red_dim", [([600, 128], 0, (1,)), ([100, 4000], 1, (0,)), ([32, 9000], 0, (0,))])
def test_sch_concat_reduce(in_shape, cat_dim, red_dim):  # :405-416
    a0, a1 = rng(61).normal(0, 0.05, in_shape).astype(np.float32), rng(62).normal(0, 0.04, in_shape).astype(np.float32)
    g = np.sum(np.concatenate([a0, a1], axis=cat_dim), red_dim, keepdims=True)
    run_graph("", lambda k: [(k.store(k.sum(k.concat([k.load(a0), k.load(a1)], cat_dim), red_dim, True)), g, 1e-4)], oracle_eps=1e-4)


@pytest.mark.parametrize("shape1, broad_shape1, shape2, cat_dim", [([1, 512], [20, 512], [4, 5, 512], 1), ([1, 512], [20, 512], [20, 4, 128], 1),
                                                                   ([1, 512], [20, 512], [20 * 512], 0)])
def test_sch_concat_reshape(shape1, broad_shape1, shape2, cat_dim):  # :419-433
    a0, a1 = rng(63).normal(0, 1, shape1).astype(np.float16), rng(64).normal(0, 1, shape2).astype(np.float16)
    g = np.concatenate([np.broadcast_to(a0, broad_shape1).reshape(shape2), a1], axis=cat_dim)
    run_graph("", lambda k: [(k.store(k.concat([k.reshape(k.broadcast(k.load(a0), broad_shape1), shape2), k.load(a1)], cat_dim)), g, 0)])


def test_sch_concat_after_casts_and_reshapes():  # :455-470
    lhs = np.full([1, 8, 512], 0.5, dtype=np.float32)
    rhs = np.full([1, 8, 1, 32, 2], -0.25, dtype=np.float32)

    def g(k):
        x1 = k.reshape(k.cast(k.reshape(k.load(rhs), [1, 8, 1, 64]), "bfloat16"), [1, 8, 64])
        return [(k.store(k.concat([k.load(lhs, "bfloat16"), x1], 2)), np.concatenate([lhs, rhs.reshape(1, 8, 64)], axis=2), 0)]
    run_graph("", g)


def test_sch_slice_concat():  # :581-617
    a0, a1, a2 = (rng(65 + i).normal(0, 1, sh).astype(np.float32) for i, sh in enumerate(([600, 300], [400, 200], [200, 200])))
    e = np.exp(np.concatenate([a0[100:500, 100:300] * np.float32(0.1) + a1, a2], axis=0))
    run_graph("", lambda k: [(k.store(k.exp(k.concat([k.add(k.slice(k.mul(k.load(a0), 0.1), [100, 100], [400, 200]), k.load(a1)), k.load(a2)], 0))), e, None)])
    b0, b1, b2 = (rng(68 + i).normal(0, 1, sh).astype(np.float32) for i, sh in enumerate(([600, 300], [100, 300], [600, 300])))
    e2 = np.concatenate([b0[100:400] * np.float32(0.1), b1], axis=0) + b2[100:500] * np.float32(0.1)

    def g(k):
        c = k.concat([k.slice(k.mul(k.load(b0), 0.1), [100, 0], [300, 300]), k.load(b1)], 0)
        return [(k.store(k.add(c, k.slice(k.mul(k.load(b2), 0.1), [100, 0], [400, 300]))), e2, None)]
    run_graph("", g)


def test_sch_slice_concat_broadcast():  # :620-636
    a0, a1, a2 = (rng(71 + i).normal(0, 1, sh).astype(np.float32) for i, sh in enumerate(([600, 200], [400, 200], [200, 200])))
    e = np.exp(np.concatenate([a0[100:500, 50:51] * np.float32(0.1) + a1, a2], axis=0))
    run_graph("", lambda k: [(k.store(k.exp(k.concat([k.add(k.slice(k.mul(k.load(a0), 0.1), [100, 50], [400, 1]), k.load(a1)), k.load(a2)], 0))), e, None)])


def test_sch_split_concat():  # :639-651
    a0 = rng(74).normal(0, 1, [500, 512]).astype(np.float32)
    e2, e3, e4 = np.split(a0 + np.float32(0.1), [200, 400])

    def g(k):
        x2, x3, x4 = k.split(k.add(k.load(a0), 0.1), 0, 200, 3)
        return [(k.store(x4), e4, None), (k.store(k.concat([k.mul(x2, 0.8), x3], 1)), np.concatenate([e2 * np.float32(0.8), e3], axis=1), None)]
    run_graph("", g)


def test_sch_diamonds_of_slices_and_concats():  # :698-760
    a0 = rng(75).normal(0, 1, [4, 600]).astype(np.float32)
    e = a0 + np.float32(0.1)

    def g1(k):
        x0 = k.add(k.load(a0), 0.1)
        s0a, _ = k.split(x0, 1, 300, 2)
        return [(k.store(k.exp(k.concat([s0a, k.slice(x0, [0, 150], [4, 300])], 1))), np.exp(np.concatenate([e[:, 0:300], e[:, 150:450]], axis=1)), None)]
    run_graph("", g1)
    b0 = np.arange(240, dtype=np.float32).reshape(4, 60)
    b1 = b0 + 1000

    def g2(k):  # slices of slices on the right
        x = k.add(k.load(b0), 0.0)
        s2 = k.slice(x, [0, 30], [4, 30])
        d1 = k.add(k.slice(s2, [0, 0], [4, 15]), k.slice(s2, [0, 15], [4, 15]))
        return [(k.store(k.add(k.slice(x, [0, 0], [4, 15]), d1)), b0[:, 0:15] + b0[:, 30:45] + b0[:, 45:60], 0)]

    def g3(k):  # on both sides
        x = k.add(k.load(b0), 0.0)
        s1, s4 = k.slice(x, [0, 0], [4, 30]), k.slice(x, [0, 30], [4, 30])
        d1 = k.add(k.slice(s1, [0, 0], [4, 15]), k.slice(s1, [0, 15], [4, 15]))
        d2 = k.add(k.slice(s4, [0, 0], [4, 15]), k.slice(s4, [0, 15], [4, 15]))
        return [(k.store(k.add(d1, d2)), b0[:, 0:15] + b0[:, 15:30] + b0[:, 30:45] + b0[:, 45:60], 0)]

    def g4(k):  # a broadcast column of the value meets the concat that holds the value
        x = k.add(k.load(b0), 0.0)
        c1 = k.concat([x, k.load(b1)], 1)
        z = k.add(k.broadcast(k.slice(x, [0, 30], [4, 1]), [4, 120]), c1)
        e_c1 = np.concatenate([b0, b1], axis=1)
        return [(k.store(z), np.broadcast_to(b0[0:4, 30:31], [4, 120]) + e_c1, 0), (k.store(c1), e_c1, 0)]
    run_graph("", g2)
    run_graph("", g3)
    run_graph("", g4)


def test_copies_of_views_with_other_shapes_do_not_share_a_launch_wrongly():
    # found by random graphs: stores of views of one value whose shapes differ (a chunk and a single element; the same
    # three elements as [1,3,1] and, permuted, as [3,1,1]) were put into one launch whose index space fitted neither
    a = rng(90).normal(0, 1, [5, 3, 24]).astype(np.float32)
    b = rng(91).normal(0, 1, [5, 3, 24]).astype(np.float32)

    def g1(k):
        x = k.add(k.load(a), k.load(b))
        parts = k.split(x, 2, 8, 3)
        return [(k.store(k.mul(parts[1], 2.0)), (a + b)[:, :, 8:16] * np.float32(2.0), None),
                (k.store(k.slice(parts[0], [4, 2, 3], [1, 1, 1])), (a + b)[4:5, 2:3, 3:4], None)]
    run_graph("", g1)
    c = rng(92).normal(0, 1, [5, 5, 128]).astype(np.float32)

    def g2(k):
        s = k.slice(k.load(c), [3, 2, 108], [1, 3, 16])
        parts = k.split(s, 2, 1, 16)
        return [(k.store(k.mul(parts[5], 2.0)), c[3:4, 2:5, 113:114] * np.float32(2.0), None),
                (k.store(k.permute(k.slice_dim(parts[7], 0, 0, 1), [1, 0, 2])), np.transpose(c[3:4, 2:5, 115:116], (1, 0, 2)), 0)]
    run_graph("", g2)
