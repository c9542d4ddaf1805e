"""GPU parity: OneHot, GatherLoad, PadStore and ElemAny, restating tests/ut/test_onehot.py, test_gather_load.py,
test_pad.py and test_element_any.py of the reference (cited per test): same shapes, axes, value classes and NumPy
expectations as there; every graph also runs on the CPU oracle. The reference's `tile(...)` calls pick a loop split of
its own code generator and do not change results, so they have no counterpart here; its gather tests are skipped
there on every architecture but one, their NumPy expectations are what is restated."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def rng(seed=0):
    return np.random.default_rng(seed)


def onehot_expect(indices, depth, axis, on_value, off_value):  # tests/ut/test_onehot.py:22-38
    axis = axis if axis >= 0 else indices.ndim + axis + 1
    outer = int(np.prod(indices.shape[:axis], dtype=np.int64))
    inner = int(np.prod(indices.shape[axis:], dtype=np.int64))
    ix = indices.reshape(outer, inner)
    out = np.full((outer, depth, inner), off_value, np.int32 if isinstance(on_value, int) else np.float32)
    for x in range(outer):
        for y in range(inner):
            out[x, ix[x, y], y] = on_value
    return out.reshape(indices.shape[:axis] + (depth,) + indices.shape[axis:])


# ---- OneHot ----

@pytest.mark.parametrize("shape1, shape2, axis, depth", [
    ([32], [32, 1], 1, 500), ([8], [8, 1], 1, 8000), ([40, 16], [40, 20, 16], 1, 20), ([40, 12], [40, 20, 12], 1, 20),
    ([4, 12], [4, 200, 1], 1, 200), ([4, 30, 12], [4, 10, 30, 1], 1, 10)])
def test_onehot_mode(shape1, shape2, axis, depth):  # tests/ut/test_onehot.py:41-67
    a = rng(1).integers(0, depth, shape1).astype(np.int32)
    b = np.full(shape2, 5.0, np.float32)
    expect = onehot_expect(a, depth, axis, 2.0, 0.0) * b
    run_graph("", lambda k: [(k.store(k.mul(k.one_hot(k.load(a), depth, axis, 2.0, 0.0, "float32"), k.load(b))), expect, None)])


@pytest.mark.parametrize("shape, axis, depth, dtype, on_value, off_value", [
    ([32], -1, 1000, "float16", 3.0, 1.0), ([32], 0, 1000, "bfloat16", 3.0, 1.0), ([4, 100], 1, 800, "float16", 3.0, 1.0),
    ([8, 512], 1, 200, "int32", 2, 0)])
def test_onehot_types(shape, axis, depth, dtype, on_value, off_value):  # :70-82
    a = rng(2).integers(0, depth, shape).astype(np.int32)
    expect = onehot_expect(a, depth, axis, on_value, off_value)
    run_graph("", lambda k: [(k.store(k.one_hot(k.load(a), depth, axis, on_value, off_value, dtype)), expect, None)])


@pytest.mark.parametrize("shape, axis", [([6, 7, 9], 0), ([6, 7, 9], 2), ([6, 7, 9], 3), ([6, 7, 9], -2), ([5], 0)])
def test_onehot_every_axis_and_indices_that_match_nothing(shape, axis):
    depth = 13
    a = rng(3).integers(-3, depth + 3, shape).astype(np.int32)  # below zero and past the depth: every position is off
    ax = axis if axis >= 0 else len(shape) + axis + 1
    want = (np.expand_dims(a, ax) == np.arange(depth).reshape([depth] + [1] * (len(shape) - ax))).astype(np.float32) * 1.5 + 0.25
    run_graph("", lambda k: [(k.store(k.one_hot(k.load(a), depth, axis, 1.75, 0.25, "float32")), want, None)])


@pytest.mark.parametrize("classes", [1000, 50000])  # rows of one round of the sweep, and of many
def test_onehot_feeds_a_reduce_and_computed_indices(classes):
    # the usual use: a cross-entropy pick, sum(one_hot(label) * logits) along the classes; indices computed in the graph
    logits = rng(4).normal(0, 1, [64, classes]).astype(np.float32)
    labels = rng(5).integers(0, classes // 2, [64]).astype(np.int32)
    want = logits[np.arange(64), labels * 2]

    def build(k):
        ix = k.mul(k.load(labels), 2)
        return [(k.store(k.sum(k.mul(k.one_hot(ix, classes, 1, 1.0, 0.0, "float32"), k.load(logits)), [1])), want, 1e-5)]

    run_graph("", build)


def test_onehot_dynamic_shape_and_depth():
    t = Tester("vector:dyn")
    ix = t.load([-1, -1], "int32")
    depth = t.int_array()
    o = t.store(t.one_hot(ix, depth, 1, 1.0, -1.0, "float32"))
    for shape, d in [((3, 40), 17), ((16, 8), 300), ((1, 1), 1)]:
        a = rng(6).integers(0, d, shape).astype(np.int32)
        t.input(ix, a)
        depth.update([d])
        t.run()
        assert np.array_equal(t.output(o), onehot_expect(a, d, 1, 1.0, -1.0)), t.das()


# ---- GatherLoad ----

@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.int32])
@pytest.mark.parametrize("src_shape, index_shape, axis", [
    ((256, 512), (129,), 0), ((16, 128, 256), (9, 33), 1), ((8, 64, 64), (65,), -1), ((4, 16, 64, 32), (5, 7), 2),
    ((4, 8, 16, 128), (3, 4, 9), -2)])
def test_gather_load_take_add(src_shape, index_shape, axis, dtype):  # tests/ut/test_gather_load.py:24-45
    r = rng(7)
    if np.issubdtype(dtype, np.integer):
        x, bias = r.integers(-7, 8, src_shape).astype(dtype), 2
    else:
        x, bias = r.normal(0, 1, src_shape).astype(dtype), 0.25
    n = src_shape[axis]
    ix = r.integers(-n, n, index_shape).astype(np.int32)
    expect = np.take(x, ix, axis=axis) + bias
    run_graph("", lambda k: [(k.store(k.add(k.gather_load(x, k.global_access(ix), axis=axis, gather_mode=1), bias)), expect, None)])


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.int32])
@pytest.mark.parametrize("src_shape, gather_size, axis", [
    ((256, 512), 129, 0), ((16, 128, 256), 33, 1), ((8, 64, 64), 65, -1), ((4, 16, 64, 32), 7, 2), ((4, 8, 16, 128), 9, -2)])
def test_gather_load_add(src_shape, gather_size, axis, dtype):  # :48-71
    r = rng(8)
    if np.issubdtype(dtype, np.integer):
        x, bias = r.integers(-7, 8, src_shape).astype(dtype), 2
    else:
        x, bias = r.normal(0, 1, src_shape).astype(dtype), 0.25
    n = src_shape[axis]
    index_shape = list(src_shape)
    index_shape[axis] = gather_size
    ix = r.integers(-n, n, index_shape).astype(np.int32)
    expect = np.take_along_axis(x, ix.astype(np.int64), axis=axis) + bias
    run_graph("", lambda k: [(k.store(k.add(k.gather_load(x, k.global_access(ix), axis=axis), bias)), expect, None)])


@pytest.mark.parametrize("src_shape, index, axis, out_shape, dtype, mode", [
    ((1, 7, 17), np.array([[1]], np.int32), 1, (7, 5, 3, 17), np.float16, 1),      # :74-95
    ((1, 6, 64), np.array([0], np.int32), 1, (6, 5, 64), np.float32, 1),
    ((1, 7, 17), np.full((1, 1, 17), 1, np.int32), 1, (7, 5, 17), np.float16, 0),   # :98-117
    ((1, 6, 64), np.zeros((1, 1, 64), np.int32), 1, (6, 5, 64), np.float32, 0)])
def test_gather_load_then_broadcast(src_shape, index, axis, out_shape, dtype, mode):
    x = ((np.arange(np.prod(src_shape)).reshape(src_shape) % 97) / 10).astype(dtype)
    picked = np.take(x, index, axis=axis) if mode == 1 else np.take_along_axis(x, index.astype(np.int64), axis=axis)
    expect = np.broadcast_to(picked, out_shape) + dtype(0.5)

    def build(k):
        y = k.gather_load(x, k.global_access(index), axis=axis, gather_mode=mode)
        return [(k.store(k.add(k.broadcast(y, list(out_shape)), 0.5)), expect, None)]

    t = run_graph("", build)
    assert "gather_load" in t.das()


def test_gather_load_clips_indices_past_either_end_and_reads_bf16_and_bool():
    x = rng(9).normal(0, 1, [10, 24]).astype(np.float32)
    ix = np.array([0, 9, 10, 1000, -10, -11, -1000, 3], np.int32)
    want_rows = np.array([0, 9, 9, 9, 0, 0, 0, 3])
    run_graph("", lambda k: [(k.store(k.gather_load(x, k.global_access(ix), axis=0, gather_mode=1)), x[want_rows], None)])
    xb = Tester.bf16_random_normal(0, 1, [10, 24])
    run_graph("", lambda k: [(k.store(k.gather_load(xb, k.global_access(ix), axis=0, dtype="bfloat16", gather_mode=1)), xb[want_rows], None)])
    m = rng(10).integers(0, 2, [10, 24]).astype(np.bool_)
    run_graph("", lambda k: [(k.store(k.gather_load(m, k.global_access(ix), axis=0, gather_mode=1)), m[want_rows], None)])


def test_gather_load_embedding_rows_feed_a_reduce_and_indices_are_computed():
    # an embedding lookup with a normalisation behind it; the row numbers are computed in the graph
    table = rng(11).normal(0, 1, [1000, 256]).astype(np.float32)
    tokens = rng(12).integers(0, 500, [4, 37]).astype(np.int32)
    rows = table[tokens * 2 + 1]
    want = rows / np.sqrt((rows.astype(np.float64) ** 2).sum(-1, keepdims=True)).astype(np.float32)

    def build(k):
        ix = k.add(k.mul(k.load(tokens), 2), 1)
        e = k.gather_load(table, ix, axis=0, gather_mode=1)
        return [(k.store(k.div(e, k.sqrt(k.sum(k.mul(e, e), [2], True)))), want, 1e-5)]

    run_graph("", build)


def test_gather_load_dynamic_shapes():
    t = Tester("vector:dyn")
    ix = t.global_access([-1], "int32")
    src = t.gather_load([-1, -1], ix, axis=0, dtype="float32", gather_mode=1)
    o = t.store(t.mul(src, 2.0))
    for rows, cols, n in [(7, 40, 5), (300, 8, 1000), (1, 1, 3)]:
        x = rng(13).normal(0, 1, [rows, cols]).astype(np.float32)
        i = rng(14).integers(-rows, rows, [n]).astype(np.int32)
        t.input(ix, i)
        t.input(src, x)
        t.run()
        assert np.array_equal(t.output(o), x[i] * np.float32(2.0)), t.das()


# ---- PadStore ----

@pytest.mark.parametrize("dtype, eps", [(np.float16, 1e-3), (np.float32, 1e-5)])
@pytest.mark.parametrize("shape, pad", [((200, 100), 128), ((200, 111), 139), ((1, 200), 8), ((111, 1), 1), ((3000, 111), 16)])
def test_pad_2d(dtype, eps, shape, pad):  # tests/ut/test_pad.py (two-dim cases)
    a = rng(15).normal(0, 1, shape).astype(dtype)

    def build(k):
        want = np.zeros((shape[0], shape[1] + pad), dtype)
        want[:, :shape[1]] = np.abs(a)
        return [(k.pad_store(k.abs(k.load(a)), pad), want, eps)]

    run_graph("", build)


@pytest.mark.parametrize("dtype, eps", [(np.float16, 1e-3), (np.float32, 1e-5)])
@pytest.mark.parametrize("shape, pad", [((1, 3, 200, 100), 128), ((1, 1, 200, 111), 139), ((4, 5, 111, 1), 1), ((33, 300, 111, 1), 16)])
def test_pad_4d(dtype, eps, shape, pad):  # :38-52 (the largest case with a tenth of its second dim)
    a = rng(16).normal(0, 1, shape).astype(dtype)

    def build(k):
        want = np.zeros(shape[:3] + (shape[3] + pad,), dtype)
        want[..., :shape[3]] = np.abs(a)
        return [(k.pad_store(k.abs(k.load(a)), pad), want, eps)]

    run_graph("", build)


@pytest.mark.parametrize("dtype, eps", [(np.float16, 1e-3), (np.float32, 1e-5)])
def test_pad_broadcast(dtype, eps):  # :55-69
    a = rng(17).normal(0, 1, (1024, 1)).astype(dtype)
    b = rng(18).normal(0, 1, (1024, 30)).astype(dtype)

    def build(k):
        want = np.zeros((1024, 45), dtype)
        want[:, :30] = a + b
        return [(k.pad_store(k.add(k.load(a), k.load(b)), 15), want, eps)]

    run_graph("", build)


# ---- ElemAny ----

@pytest.mark.parametrize("mask", [1, 0])
@pytest.mark.parametrize("shape", [(1024, 32), (127,), (100, 100), (23, 23)])
def test_element_any(mask, shape):  # tests/ut/test_element_any.py:22-35
    a = np.full(shape, mask, np.float32)
    run_graph("", lambda k: [(k.store(k.element_any(k.load(a))), np.array([mask], np.float32), 0)])


def test_element_any_one_element_set():  # :38-50, :66-78
    a = np.zeros([127, 127], np.float32)
    a[11, 11] = 1
    run_graph("", lambda k: [(k.store(k.element_any(k.abs(k.load(a)))), np.array([1], np.float32), 0)])
    m = np.zeros([256, 32, 64], np.bool_)
    m[1, 1, 1] = True
    run_graph("", lambda k: [(k.store(k.element_any(k.cast(k.load(m), "float32"))), np.array([1], np.float32), 0)])


@pytest.mark.parametrize("n", [1001, 3184, 5231, 128 * 9 + 20, 101 * 9 + 20, 501 * 10])
def test_element_any_nothing_set(n):  # :53-63, :81-97
    a = np.full([n], 1.0, np.float32)
    run_graph("", lambda k: [(k.store(k.element_any(k.sub(k.add(k.load(a), 1.0), 2.0))), np.array([0], np.float32), 0)])
