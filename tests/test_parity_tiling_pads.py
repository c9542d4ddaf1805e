"""GPU parity: the graphs of the reference's tests that probe how its tile machine cuts and pads shapes
(tests/ut/test_tiling.py, test_pass_insert_removepad.py, test_pass_compact_peak_liveness.py,
test_pass_double_buffer.py, test_pass_reorder_load.py, test_pass_reorder_store.py). Those tests check numbers and
then the reference's own graph listing after a pass; the numbers are what carries over. Here every graph runs
through the C ABI on the GPU with the same shapes, element types, pass names and tiling hints (accepted, without
effect: there are no tiles), against the oracle and the NumPy expectation the reference's test states. Shapes
with innermost extents of 1, 2, 3, 5, 24, 77 and 80 are the point: rows far from a multiple of a lane's sixteen
bytes, broadcasts along inner and outer axes at once."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def hint(k, name, *args):
    """A scheduling hint of the reference's harness (tile, set_passes, spec_next): the oracle has no such thing."""
    f = getattr(k, name, None)
    if f is not None:
        f(*args)


# ---- tests/ut/test_tiling.py ----

@pytest.mark.parametrize("dim", [1024, 1023])
def test_row_broadcast_over_512_rows(dim):
    a, b = np.full([1, dim], 0.5, np.float32), np.full([512, dim], 0.2, np.float32)

    def build(k):
        return [(k.store(k.add(k.broadcast(k.load(a), [512, dim]), k.load(b))), np.float32(0.5) + np.float32(0.2), None)]
    run_graph("vector", build)


@pytest.mark.parametrize("rows", [160, 16000])
def test_innermost_broadcast_to_80(rows):
    rng = np.random.default_rng(rows)
    b = rng.standard_normal([rows, 39, 1], dtype=np.float32)

    def build(k):
        return [(k.store(k.broadcast(k.load(b), [rows, 39, 80])), np.broadcast_to(b, (rows, 39, 80)), 0)]
    run_graph("vector", build, oracle=rows < 1000)


def test_outer_broadcast_of_whole_planes():
    rng = np.random.default_rng(5)
    a = rng.standard_normal([2, 1, 64, 1024], dtype=np.float32)

    def build(k):
        return [(k.store(k.broadcast(k.load(a), [2, 96, 64, 1024])), np.broadcast_to(a, (2, 96, 64, 1024)), 0)]
    run_graph("vector", build, oracle=False)


@pytest.mark.parametrize("src,dst,tiles", [
    ([2, 1, 512], [2, 3, 512], [(2, 2, 2), (1, 1, 3), (0, 0, 4)]),
    ([2, 1, 4, 1, 512], [2, 3, 4, 6, 512], [(4, 4, 2), (3, 3, 3), (2, 2, 4), (1, 1, 3)]),
    ([2, 1, 4, 1, 512], [2, 3, 4, 5, 512], [(4, 4, 2), (3, 3, 3), (2, 2, 4), (1, 1, 5), (0, 1, 2)]),
])
def test_broadcast_with_tiling_hints(src, dst, tiles):
    rng = np.random.default_rng(len(dst))
    a = rng.standard_normal(src, dtype=np.float32)

    def build(k):
        st = k.store(k.broadcast(k.load(a), dst))
        for h in tiles:
            hint(k, "tile", *h)
        return [(st, np.broadcast_to(a, dst), 0)]
    run_graph("vector", build)


def test_scalar_quotient_broadcast_twice():
    # one number divided by one number, broadcast to a column, reshaped, broadcast to 5120 x 21128 and multiplied
    one = np.full([1], 1.1, np.float32)
    col = np.full([5120], 1.1, np.float32)
    big = np.ones([5120, 21128], np.float32)

    def build(k):
        y = k.broadcast(k.div(k.load(one), k.load(one)), [5120])
        r = k.mul(k.mul(k.load(col), y), -1.0)
        m = k.mul(k.broadcast(k.reshape(r, [5120, 1]), [5120, 21128]), k.load(big))
        return [(k.store(m), np.float32(-1.1), 1e-6)]
    run_graph("split", build, oracle=False)


def test_one_element_and_no_dims():
    def build(k):
        a = k.store(k.sqrt(k.load(np.full([1, 1], 0.04, np.float32))))
        b = k.store(k.mul(k.full(0.2, [], "float32"), 0.3))
        return [(a, np.sqrt(np.float32(0.04)), 1e-6), (b, np.float32(0.2) * np.float32(0.3), 1e-6)]
    run_graph("split", build)


@pytest.mark.parametrize("dim1,dim2", [([2, 8], [16]), ([16], [2, 8]), ([2, 16], [2, 4, 4])])
def test_reshape_of_outer_axes_behind_a_broadcast(dim1, dim2):
    inner = [10240]
    a = np.full(dim1 + [1], 0.3, np.float32)

    def build(k):
        y = k.mul(k.broadcast(k.load(a), dim1 + inner), 0.6)
        return [(k.store(k.sqrt(k.reshape(y, dim2 + inner))), np.sqrt(np.float32(0.3) * np.float32(0.6)), 1e-6)]
    run_graph("split", build)


def test_two_stores_of_different_extent():
    g0, g1 = np.full([32, 1], 0.1, np.float32), np.full([32, 1024], 0.1, np.float32)

    def build(k):
        a, b = k.load(g0), k.load(g1)
        return [(k.store(k.add(a, b)), np.full([32, 1024], np.float32(0.1) + np.float32(0.1)), None),
                (k.store(k.add(a, 0.2)), np.full([32, 1], np.float32(0.1) + np.float32(0.2)), None)]
    run_graph("vector", build)


# ---- tests/ut/test_pass_insert_removepad.py ----

@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_box_overlap_with_innermost_two(dtype):
    # [32,26,26,3,1,2] against [32,1,1,1,50,2]: the overlap of two sets of boxes, broadcast along four axes
    rng = np.random.default_rng(11)
    a, b = (rng.standard_normal([32, 26, 26, 3, 1, 2]).astype(dtype) for _ in range(2))
    c, d = (rng.standard_normal([32, 1, 1, 1, 50, 2]).astype(dtype) for _ in range(2))
    half = dtype(0.5)
    gold = np.maximum(np.minimum(a * half + b, c * half + d) - np.maximum(b - half * a, d - half * c), dtype(0))

    def build(k):
        xa, xb, xc, xd = k.load(a), k.load(b), k.load(c), k.load(d)
        ha, hc = k.mul(xa, 0.5), k.mul(xc, 0.5)
        lo = k.minimum(k.add(xb, ha), k.add(xd, hc))
        hi = k.maximum(k.sub(xb, ha), k.sub(xd, hc))
        st = k.store(k.maximum(k.sub(lo, hi), 0))
        hint(k, "set_passes", "InsertRemovePad")
        return [(st, gold, 2e-3 if dtype is np.float16 else 1e-6)]
    run_graph("vector", build, oracle=False)


def test_column_and_44_wide_rows():
    rng = np.random.default_rng(12)
    a, b = rng.standard_normal([32, 1], dtype=np.float32), rng.standard_normal([32, 44], dtype=np.float32)

    def build(k):
        x, y = k.load(a), k.load(b)
        out = [(k.store(k.mul(x, 0.5)), a * np.float32(0.5), None), (k.store(k.add(x, y)), a + b, None)]
        hint(k, "set_passes", "InsertRemovePad")
        return out
    run_graph("vector", build)


def test_broadcast_to_five_then_to_32_rows():
    n = 40 + 39
    b = np.full([n, 1, 1], 0.3, np.float32)

    def build(k):
        z = k.add(k.broadcast(k.load(b), [n, 1, 5]), 0.1)
        st = k.store(k.broadcast(z, [n, 32, 5]))
        hint(k, "set_passes", "InsertRemovePad")
        return [(st, np.float32(0.3) + np.float32(0.1), None)]
    run_graph("vector", build)


def test_fp16_rows_of_77_against_a_column():
    rng = np.random.default_rng(14)
    a = (rng.standard_normal([20, 4096, 1]) * 0.1).astype(np.float32)
    b, c = ((rng.standard_normal([20, 4096, 77]) * 0.1).astype(np.float16) for _ in range(2))
    gold = (c - a.astype(np.float16)) * b * np.float16(1.2)

    def build(k):
        y = k.mul(1.2, k.mul(k.load(b), k.sub(k.load(c), k.cast(k.load(a), "float16"))))
        st = k.store(y)
        hint(k, "set_passes", "InsertRemovePad")
        return [(st, gold, 2e-3)]
    run_graph("vector", build, oracle=False)


def test_masked_softmax_over_rows_of_204_in_stages():
    # tests/ut/test_pass_insert_removepad.py:94-135: a speculative vector kernel in three stages
    rng = np.random.default_rng(15)
    shape = [80, 204, 204]
    mask = rng.uniform(0, 1, shape) > 0.5
    lowest = np.array(-3.4028234663852886e38, dtype=np.float32)
    x = rng.standard_normal(shape, dtype=np.float32)
    w = np.where(mask, lowest, x / np.float32(8.0))
    e = np.exp(w - w.max(axis=2, keepdims=True))
    gold = e / e.sum(axis=2, keepdims=True)

    def build(k):
        where = k.select(k.load(mask), k.broadcast(k.load(lowest), shape), k.div(k.load(x), 8.0))
        top = k.max(where, (2,), True)
        hint(k, "spec_next")
        ex = k.exp(k.sub(where, k.broadcast(top, shape)))
        total = k.sum(ex, (2,), True)
        hint(k, "spec_next")
        st = k.store(k.div(ex, k.broadcast(total, shape)))
        hint(k, "set_passes", "InsertRemovePad")
        return [(st, gold, 1e-4)]
    run_graph("vector:spec", build, oracle=False)


def test_quotient_by_a_column_stored_twice():
    rng = np.random.default_rng(16)
    a0 = rng.standard_normal([1, 4096, 4], dtype=np.float32)
    a1 = np.abs(rng.standard_normal([1, 4096, 1], dtype=np.float32) * 10) + np.float32(1e-4)

    def build(k):
        q = k.div(k.load(a0), k.load(a1))
        out = [(k.store(q), a0 / a1, 1e-4), (k.store(k.cast(k.mul(q, 2.0), "bfloat16")), a0 / a1 * 2, 1e-2)]
        hint(k, "set_passes", "InsertRemovePad")
        return out
    run_graph("vector", build)


@pytest.mark.parametrize("shape1,shape2", [((32, 1, 4096, 1), (32, 1, 1, 24)), ((1024, 64, 1), (1024, 1, 5)),
                                           ((2, 800, 64, 1), (1, 800, 1, 5))])
@pytest.mark.parametrize("determ", [False, True])
def test_sum_over_the_outermost_axis_behind_a_cast(shape1, shape2, determ):
    rng = np.random.default_rng(len(shape1) + shape1[0])
    a, b = rng.standard_normal(shape1).astype(np.float16), rng.standard_normal(shape2).astype(np.float16)
    gold = np.sum((a + b).astype(np.float32), axis=0)

    def build(k):
        st = k.store(k.sum(k.cast(k.add(k.load(a), k.load(b)), "float32"), (0,), False))
        hint(k, "set_passes", "InsertRemovePad")
        return [(st, gold, 1e-4)]
    Tester.set_deterministic(determ)
    try:
        run_graph("vector", build, oracle_eps=1e-4)
    finally:
        Tester.set_deterministic(False)


def test_dynamic_shapes_with_innermost_3_and_32():
    t = Tester("vector:dyn")
    x0, x1 = t.load([-1, -1, -1], "float32"), t.load([-1, -1, -1], "float32")
    s = t.add(x0, x1)
    out1 = t.store(s)
    out2 = t.store(t.sum(t.mul(s, 0.5), [2], True))
    t.set_passes("InsertRemovePad")
    rng = np.random.default_rng(17)
    for shape1, shape2 in [([40, 2000, 3], [40, 1, 3]), ([40, 2000, 32], [40, 2000, 32]), ([2000, 5, 32], [1, 5, 32])]:
        a = (rng.standard_normal(shape1) * 0.1).astype(np.float32)
        b = (rng.standard_normal(shape2) * 0.1).astype(np.float32)
        t.input(x0, a)
        t.input(x1, b)
        t.run()
        assert t.check(out1, a + b)
        assert t.check(out2, np.sum((a + b) * np.float32(0.5), (2,), keepdims=True), 1e-4)


# ---- the graphs of the liveness, double-buffer and reorder tests: many values alive at once, several stores ----

@pytest.mark.parametrize("ker", ["vector", "vector:dyn"])
def test_five_stores_of_one_load(ker):
    a = np.full([128, 32], 2, np.float16)
    f = np.float16
    g1 = np.exp(f(2))
    g2 = np.log(g1)
    g3, g4 = g2 + f(2), g2 + g1
    golds = [np.exp(g4), abs(g4), g2 + f(2), g3 + np.sqrt(g4), np.sqrt(g3)]

    def build(k):
        x0 = k.load(a)
        x1 = k.exp(x0)
        x2 = k.log(x1)
        x3, x4 = k.add(x2, x0), k.add(x2, x1)
        outs = [k.exp(x4), k.abs(x4), k.add(x2, x0), k.add(x3, k.sqrt(x4)), k.sqrt(x3)]
        stores = [(k.store(o), np.float32(g), 2e-3) for o, g in zip(outs, golds)]
        hint(k, "set_passes", "PrintPeakLive", "CompactPeakLiveness", "PrintPeakLive")
        return stores
    run_graph(ker, build)


def test_chain_of_logarithms_with_four_stores():
    a = np.full([128, 32], 23, np.float16)

    def build(k):
        x0 = k.load(a)
        x1 = k.log(x0)
        x2 = k.log(x1)
        x3 = k.log(x2)
        x4, x5, x6 = k.add(x2, x3), k.log(x2), k.add(x2, x0)
        outs = [k.log(x1), k.add(x2, x5), k.add(x3, x4), k.log(x6)]
        stores = [(k.store(o), None, None) for o in outs]
        hint(k, "set_passes", "PrintPeakLive", "CompactPeakLiveness", "PrintPeakLive")
        return stores
    run_graph("vector", build)


def test_select_between_two_branches_with_casts():
    a = np.full([128, 32], 23, np.float16)

    def build(k):
        x0 = k.load(a)
        x1, x2 = k.log(x0), k.reciprocal(x0)
        x3 = k.add(x1, x2)
        both = k.add(k.cast(x1, "float32"), k.cast(x3, "float32"))
        pick = k.select(k.greater(x1, x2), x2, x3)
        stores = [(k.store(pick), None, None), (k.store(both), None, None)]
        hint(k, "set_passes", "PrintPeakLive", "CompactPeakLiveness", "PrintPeakLive")
        return stores
    run_graph("vector", build)


@pytest.mark.parametrize("shape", [[1000, 2000], [128]])
def test_two_loads_four_operators(shape):
    a = np.full(shape, 2, np.float16)

    def build(k):
        x0, x1 = k.load(a), k.load(a.copy())
        st = k.store(k.mul(k.add(k.add(x0, 0.1), k.add(x1, 0.1)), x0))
        hint(k, "set_passes", "VectorDoubleBuffer")
        return [(st, np.float16(8.4), 2e-3)]
    run_graph("vector", build)


@pytest.mark.parametrize("ker", ["vector", "vector:dyn"])
def test_loads_between_operators_and_stores_of_intermediates(ker):
    a, b, c = (np.full([8], v, np.float16) for v in (9, 2, 3))

    def build(k):
        x2 = k.sqrt(k.load(a))
        x4 = k.add(k.load(b), x2)
        x6 = k.add(x4, k.load(c))
        hint(k, "set_passes", "ReorderLoad", "ReorderStore")
        return [(k.store(x6), np.float16(8.0), None), (k.store(x2), np.float16(3.0), None), (k.store(x4), np.float16(5.0), None)]
    run_graph(ker, build)


def test_store_of_a_value_computed_before_an_unrelated_chain():
    a, b = np.full([8], 2, np.float16), np.full([8], 9, np.float16)

    def build(k):
        x1, x2 = k.load(a), k.load(b)
        x3 = k.reciprocal(x1)
        x5 = k.add(k.sqrt(x2), x1)
        hint(k, "set_passes", "ReorderStore")
        return [(k.store(x5), np.float16(5.0), None), (k.store(x3), np.float16(0.5), None)]
    run_graph("vector", build)


def test_load_used_twice_beside_a_load_used_once():
    a, b = np.full([8], 4, np.float16), np.full([8], 9, np.float16)

    def build(k):
        x1, x2 = k.load(a), k.load(b)
        hint(k, "set_passes", "ReorderLoad")
        return [(k.store(k.add(k.add(x1, x2), k.mul(x1, 0.5))), np.float16(15.0), None)]
    run_graph("vector", build)
