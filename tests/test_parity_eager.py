"""GPU parity: the graph-cutting cases of the reference's tests/ut/test_eager_fusion.py (cited per test), run
through the "eager" kernel type: same shapes, input distributions, NumPy expectations and tolerances; every
graph also runs on the CPU oracle. What these graphs probe is where a graph is cut into launches and how values
cross the cuts (workspace, re-use of a user's output, broadcasts and reduces on either side of a cut)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["eager", "eager:unify_ws", "eager:lazy", "eager:lazy,unify_ws"])
def test_split_end(mode):  # tests/ut/test_eager_fusion.py:22-41: reduce -> broadcast; the kernel object is reused
    g0, g1, g2 = np.full([32, 1], 0.1, np.float32), np.full([32, 1024], 0.1, np.float32), np.full([10, 1024], 0.1, np.float32)
    expect = np.sqrt(np.sum((g0 + g1) * 2.0, (0,), keepdims=True) - g2)
    t = Tester(mode)
    for _ in range(2):
        x = t.mul(t.add(t.load(g0), t.load(g1)), 2.0)
        x = t.sqrt(t.sub(t.sum(x, [0], True), t.load(g2)))
        t.store_expect(x, expect)
        assert t.run_check()
        t.reset()


def test_split_middle():  # :44-66
    g0, g1, g2 = np.full([32, 1], 0.1, np.float32), np.full([32, 1024], 0.1, np.float32), np.full([32, 512], 0.1, np.float32)
    ex = g0 + 0.1

    def g(k):
        x = k.add(k.load(g0), 0.1)
        y = k.add(x, k.load(g1))
        z = k.sum(k.add(k.load(g2), x), [1], True)
        sz = k.store(z)
        return [(sz, np.sum(g2 + ex, (1,), keepdims=True), None), (k.store(k.mul(y, 0.1)), (ex + g1) * 0.1, None)]
    run_graph("eager", g)


def test_split_join():  # :69-93
    g0, g1, g2 = np.full([32, 1], 0.1, np.float32), np.full([32, 1024], 0.1, np.float32), np.full([32, 512], 0.1, np.float32)
    ex = g0 + 0.1

    def g(k):
        x = k.add(k.load(g0), 0.1)
        y = k.add(x, k.load(g1))
        z = k.sum(k.add(k.load(g2), x), [1], True)
        return [(k.store(k.mul(k.add(z, y), 0.1)), ((ex + g1) + np.sum(g2 + ex, (1,), keepdims=True)) * 0.1, None)]
    run_graph("eager", g)


@pytest.mark.parametrize("shape1,shape2", [((1, 1280, 28, 36), (1, 1280, 1, 1)), ((1, 8, 28, 512), (1, 8, 1, 1)),
                                           ((1, 1000, 28, 128), (1, 1000))])
def test_disconnected_graphs(shape1, shape2):  # :96-113
    rng = np.random.default_rng(shape1[1])
    x0, x1 = rng.normal(0, 1, shape1).astype(np.float16), rng.normal(0, 1, shape1).astype(np.float16)
    x2, x3 = rng.normal(0, 1, shape2).astype(np.float16), rng.normal(0, 1, shape2).astype(np.float16)

    def g(k):
        a = k.add(k.load(x0), k.load(x1))
        b = k.add(k.load(x2), k.load(x3))
        return [(k.store(a), x0 + x1, None), (k.store(b), x2 + x3, None)]
    run_graph("eager", g, min_launches=2)


def test_dead_node():  # :116-131
    g0, g1, g2 = np.full([32, 512], 0.1, np.float32), np.full([32, 512], 0.2, np.float32), np.full([32, 512], 0.3, np.float32)
    t = Tester("eager")
    t.sub(t.load(g0), t.load(g1))  # dead
    t.store_expect(t.mul(t.add(t.load(g2), 0.1), 2.0), (0.3 + 0.1) * 2.0)
    assert t.run_check()
    assert t.das().count("load.") == 1


def test_split_load():  # :134-150
    rng = np.random.default_rng(1)
    g0, g1, g2 = (rng.normal(0, 1, s).astype(np.float32) for s in ((4, 32), (10, 4, 32), (12, 4, 32)))

    def g(k):
        x0 = k.load(g0)
        return [(k.store(k.add(x0, k.load(g1))), g0 + g1, None), (k.store(k.add(x0, k.load(g2))), g0 + g2, None)]
    run_graph("eager", g)


def test_split_load_reduce():  # :153-166
    rng = np.random.default_rng(2)
    g0, g1, g2 = (rng.normal(0, 1, s).astype(np.float32) for s in ((1, 4, 1024), (1, 1, 1024), (12, 4, 1024)))

    def g(k):
        x0 = k.add(k.load(g0), k.load(g1))
        x1 = k.sum(k.load(g2), (0,), True)
        return [(k.store(x0), g0 + g1, None), (k.store(x1), np.sum(g2, axis=(0,), keepdims=True), None)]
    run_graph("eager", g)


def test_stop_fuse_reduce():  # :169-186
    rng = np.random.default_rng(3)
    a0, a3, a5 = rng.normal(0, 0.1, [428, 16, 8]).astype(np.float32), rng.normal(0, 0.1, (1,)).astype(np.float32), \
        rng.normal(0, 0.1, [428, 16]).astype(np.float32)

    def g(k):
        x2 = k.sum(k.abs(k.load(a0)), (2,), False)
        return [(k.store(k.add(k.load(a5), k.mul(x2, k.load(a3)))), a5 + np.sum(np.abs(a0), axis=2) * a3, None)]
    run_graph("eager", g)


def test_reduce_multi_user():  # :189-203
    rng = np.random.default_rng(4)
    a0, a4 = rng.normal(0, 0.1, [428, 16, 8]).astype(np.float32), rng.normal(0, 0.1, [428, 1]).astype(np.float32)
    e2 = np.sum(np.abs(a0), axis=2)

    def g(k):
        x2 = k.sum(k.abs(k.load(a0)), (2,), False)
        return [(k.store(k.add(k.mul(x2, x2), k.load(a4))), e2 * e2 + a4, None)]
    run_graph("eager", g)


@pytest.mark.parametrize("mode", ["eager", "eager:unify_ws"])
@pytest.mark.parametrize("shape_a,shape_b", [([128, 1024], [1024, 256]), ([128, 500], [500, 256]), ([128, 1024], [1024, 500]),
                                             ([1024, 1, 256], [256, 512])])
def test_mm(mode, shape_a, shape_b):  # :206-227 (the 4096x34816x2560 case is left to the matmul parity file's sizes)
    np.random.seed(5)
    a = Tester.fast_random_normal(0, 0.01, shape_a).astype(np.float16)
    b = Tester.fast_random_normal(0, 0.01, shape_b).astype(np.float16)

    def g(k):
        x2 = k.matmul(k.add(k.load(a), 0.01), k.load(b), False, False)
        return [(k.store(k.add(x2, 1.0)), np.matmul((a + np.float16(0.01)).astype(np.float32), b.astype(np.float32)) + 1.0, 2e-3)]
    run_graph(mode, g)


def test_mm_bias():  # :230-258, fp16 and bf16
    rng = np.random.default_rng(6)
    a, b, c = rng.normal(0, 0.01, [256, 512]), rng.normal(0, 0.01, [512, 256]), rng.normal(0, 0.01, [256])
    a16, b16, c16 = a.astype(np.float16), b.astype(np.float16), c.astype(np.float16)
    run_graph("eager", lambda k: [(k.store(k.matmul(k.load(a16), k.load(b16), False, False, k.load(c16))),
                                   np.matmul(a16.astype(np.float32), b16.astype(np.float32)) + c16, 2e-3)])
    a32, b32, c32 = a.astype(np.float32), b.astype(np.float32), c.astype(np.float32)
    run_graph("eager", lambda k: [(k.store(k.matmul(k.load(a32, "bfloat16"), k.load(b32, "bfloat16"), False, False,
                                                    k.load(c32, "bfloat16"))), np.matmul(a32, b32) + c32, 5e-3)])


def test_kernel_object_reuse():  # :261-287, :305-322: vector, matmul, vector through one kernel object
    rng = np.random.default_rng(7)
    t = Tester("eager")
    a = rng.normal(0, 0.1, [256, 2048]).astype(np.float32)
    t.store_expect(t.add(t.sum(t.load(a), (0,), True), 0.2), np.sum(a, (0,), keepdims=True) + 0.2, 1e-4)
    assert t.run_check()
    t.reset()
    a16, b16 = rng.normal(0, 0.01, [256, 512]).astype(np.float16), rng.normal(0, 0.01, [512, 256]).astype(np.float16)
    t.store_expect(t.add(t.matmul(t.load(a16), t.load(b16), False, False), 0.1),
                   np.matmul(a16.astype(np.float32), b16.astype(np.float32)) + 0.1, 2e-3)
    assert t.run_check()
    t.reset()
    a = rng.normal(0, 0.1, [256, 512]).astype(np.float32)
    t.store_expect(t.add(t.add(t.load(a), 0.2), 0.2), a + 0.4)
    assert t.run_check()
    t.reset()
    x0, x1, x2, x3 = (np.full(s, v, np.float32) for s, v in (([32, 1024], 0.1), ([32, 1024], 0.2), ([10, 1024], 0.4), ([10, 1024], 0.1)))
    for _ in range(3):  # :290-302
        t.store_expect(t.mul(t.load(x0), t.load(x1)), 0.02)
        t.store_expect(t.sub(t.load(x2), t.load(x3)), 0.3)
        assert t.run_check()
        t.reset()


def test_long_chain():  # :325-335: 200 adds behind one load
    ax = np.random.default_rng(8).normal(0, 0.1, [512, 512]).astype(np.float32)
    bx = np.full([1, 512], 0.01, np.float32)

    def g(k):
        a, b = k.load(ax), k.load(bx)
        for _ in range(200):
            a = k.add(a, b)
        return [(k.store(a), ax + 0.01 * 200, 1e-4)]
    run_graph("eager", g)


def test_workspace_inplace():  # :338-350
    rng = np.random.default_rng(9)
    a, b = rng.normal(0, 0.1, [128, 1024]).astype(np.float16), rng.normal(0, 0.1, [1, 1024]).astype(np.float32)

    def g(k):
        x0 = k.cast(k.load(a), "float32")
        s0 = k.store(k.cast(k.sum(x0, (0,), False), "float16"))
        return [(s0, np.sum(a.astype(np.float32), axis=0).astype(np.float16), 2e-3),
                (k.store(k.mul(k.load(b), x0)), b * a.astype(np.float32), None)]
    run_graph("eager", g)


def test_load_reuse():  # :353-369
    rng = np.random.default_rng(10)
    ax, bx, cx = rng.normal(0, 0.1, [288]).astype(np.float32), rng.normal(0, 0.1, [1]).astype(np.float32), \
        rng.normal(0, 0.1, [864, 1152]).astype(np.float32)

    def g(k):
        x1 = k.load(bx)
        x2 = k.mul(k.load(ax), x1)
        s2 = k.store(x2)
        s4 = k.store(k.add(k.load(cx), x1))
        return [(s2, ax * bx, None), (s4, cx + bx, None), (k.store(k.add(x2, 0.1)), ax * bx + 0.1, None)]
    run_graph("eager", g)


def test_parallel_areas():  # :391-435
    run_graph("eager", lambda k: [(k.store(k.add(k.load(np.full([32, 1024], 0.1, np.float32)), 1.0)), 1.1, None),
                                  (k.store(k.add(k.load(np.full([32, 1024], 0.1, np.float32)), 2.0)), 2.1, None)])

    def g2(k):
        x1 = k.sum(k.load(np.full([10, 1024], 0.1, np.float32)), (0,), True)
        return [(k.store(k.add(k.load(np.full([16, 1024], 0.2, np.float32)), x1)), 1.2, None),
                (k.store(k.add(k.load(np.full([17, 1024], 0.3, np.float32)), x1)), 1.3, None)]
    run_graph("eager", g2)

    def g3(k):
        x1 = k.sum(k.load(np.full([4, 5, 3, 1024], 0.1, np.float32)), (0,), True)
        return [(k.store(k.add(k.sum(x1, (1,), True), k.sum(x1, (2,), True))), 3.2, None)]
    run_graph("eager", g3)


def test_matmul_then_two_areas():  # :438-477 (cv_0, cv_1), :480-495 (cv_2)
    rng = np.random.default_rng(11)
    a, b = rng.normal(0, 0.01, [256, 512]).astype(np.float16), rng.normal(0, 0.01, [512, 256]).astype(np.float16)
    c = rng.normal(0, 0.01, [2, 256, 256]).astype(np.float16)
    e2 = np.matmul(a.astype(np.float32), b.astype(np.float32)).astype(np.float16)

    def g0(k):
        x3 = k.add(k.matmul(k.load(a), k.load(b), False, False), 0.1)
        return [(k.store(k.add(x3, 0.1)), e2 + np.float16(0.2), None), (k.store(k.sub(x3, 0.05)), e2 + np.float16(0.05), None)]
    run_graph("eager", g0)

    def g1(k):
        x2 = k.matmul(k.load(a), k.load(b), False, False)
        s4 = k.store(k.add(k.add(x2, 0.1), 0.1))
        return [(s4, e2 + np.float16(0.2), None), (k.store(k.sub(x2, k.load(c))), e2 - c, None)]
    run_graph("eager", g1)

    def g2(k):
        x0, x1 = k.mul(k.load(a), 1.2), k.mul(k.load(b), 0.8)
        s1 = k.store(x1)
        return [(s1, b * np.float16(0.8), None),
                (k.store(k.matmul(x0, x1, False, False)),
                 np.matmul((a * np.float16(1.2)).astype(np.float32), (b * np.float16(0.8)).astype(np.float32)).astype(np.float16), None)]
    run_graph("eager", g2)


def test_matmul_same_input():  # :498-523
    rng = np.random.default_rng(12)
    a, b = rng.normal(0, 0.01, [1024, 1024]).astype(np.float16), rng.normal(0, 0.01, [1024, 1024]).astype(np.float16)
    a32 = a.astype(np.float32)
    run_graph("eager", lambda k: (lambda x0: [(k.store(k.add(k.matmul(x0, x0, False, False), 0.1)),
                                               np.matmul(a32, a32).astype(np.float16) + np.float16(0.1), None)])(k.load(a)))

    def g(k):
        x1 = k.load(b)
        return [(k.store(k.add(k.matmul(k.load(a), x1, False, False), x1)), np.matmul(a32, b.astype(np.float32)).astype(np.float16) + b, None)]
    run_graph("eager", g)


@pytest.mark.parametrize("shape_a,shape_b,shape_c", [([1024, 512], [512, 1024], [1, 1024]), ([512, 512], [512, 1024], [512, 1]),
                                                     ([2, 4, 512, 512], [512, 256], [2, 1, 512, 1]),
                                                     ([2, 4, 512, 512], [2, 1, 512, 256], [256]),
                                                     ([1024, 1, 256], [256, 512], [1024, 1, 512]),
                                                     ([1024, 1, 256], [256, 512], [1, 1, 512]),
                                                     ([1024, 1, 256], [256, 512], [1024, 1, 1]),
                                                     ([4, 128, 1, 256], [256, 512], [4, 1, 1, 512])])
def test_matmul_broadcast_epilogue(shape_a, shape_b, shape_c):  # :526-549
    rng = np.random.default_rng(len(shape_a) * 100 + shape_c[-1])
    a, b, c = (rng.normal(0, 0.01, s).astype(np.float16) for s in (shape_a, shape_b, shape_c))
    e2 = np.matmul(a.astype(np.float32), b.astype(np.float32)).astype(np.float16)

    def g(k):
        x2 = k.matmul(k.load(a), k.load(b), False, False)
        x4 = k.add(k.load(c), 0.1)
        s5 = k.store(k.add(x2, x4))
        return [(s5, e2 + (c + np.float16(0.1)), None), (k.store(x4), c + np.float16(0.1), None)]
    run_graph("eager", g)


def test_multi_parallel_area():  # :552-577
    rng = np.random.default_rng(13)
    i0, i1, i2, i3 = rng.random([2, 3, 4]).astype(np.float32), rng.random([1]).astype(np.float32), \
        rng.random([2, 3, 4]).astype(np.float32), rng.random([1]).astype(np.float32)

    def g(k):
        t4 = k.mul(k.cast(k.load(i0), "float16"), k.cast(k.load(i1), "float16"))
        s5 = k.store(t4)
        t7 = k.cast(k.load(i2), "float16")
        s8 = k.store(t7)
        t10 = k.cast(k.load(i3), "float16")
        s11 = k.store(t10)
        s14 = k.store(k.cast(k.mul(t7, t10), "float16"))
        return [(s5, i0.astype(np.float16) * i1.astype(np.float16), None), (s8, i2.astype(np.float16), None),
                (s11, i3.astype(np.float16), None), (s14, i2.astype(np.float16) * i3.astype(np.float16), None)]
    run_graph("eager", g)


def test_many_outputs():  # :580-596: fifty doublings, every one stored
    def g(k):
        x = k.load(np.full([5, 4], 0.1, np.float32))
        out, e = [], 0.1
        for _ in range(50):
            x = k.add(x, x)
            e *= 2
            out.append((x, e))
        return [(k.store(v), np.float32(ev), 1e-5 * ev) for v, ev in out]
    run_graph("eager", g)


def test_reduce_depends_on_reduce():  # :599-614
    a = np.random.default_rng(14).normal(0, 0.1, [1, 32, 2, 4]).astype(np.float32)
    e2 = np.sum(a + 0.125, axis=(0, 2, 3), keepdims=True)

    def g(k):
        x0 = k.load(a)
        x2 = k.sum(k.add(x0, 0.125), (0, 2, 3), True)
        s2 = k.store(x2)
        x5 = k.sum(k.mul(k.sub(x0, x2), -0.125), (0, 2, 3), False)
        return [(s2, e2, None), (k.store(x5), np.sum((a - e2) * (-0.125), axis=(0, 2, 3)), None)]
    run_graph("eager", g)


@pytest.mark.parametrize("mode", ["eager", "eager:unify_ws"])
def test_operators_without_a_store_are_skipped(mode):  # :617-632
    a = np.random.default_rng(15).normal(0, 0.1, [1, 32, 2, 4]).astype(np.float32)
    t = Tester(mode)
    x1 = t.add(t.load(a), 0.125)
    t.store_expect(t.sum(x1, (0, 2, 3), True), np.sum(a + 0.125, axis=(0, 2, 3), keepdims=True))
    t.add(t.sum(t.mul(t.sqrt(x1), -0.125), (0, 2, 3), False), 0.02)
    assert t.run_check()
    assert t.num_launches() == 1


def test_store_inplace():  # :635-651
    a = np.random.default_rng(16).normal(0, 0.1, [64, 128]).astype(np.float32)
    t = Tester("eager")
    x2 = t.mul(t.sum(t.load(a), (1,), True), 0.5)
    x4 = t.store_expect(t.add(x2, x2), np.sum(a, axis=(1,), keepdims=True) * 0.5 * 2)
    t.set_store_inplace(x4)
    assert t.run_check()


def test_select_across_areas():  # :654-671
    rng = np.random.default_rng(17)
    a, b, c = rng.normal(0, 0.1, [64, 128]).astype(np.float32), rng.normal(0, 0.1, [64, 128]).astype(np.float32), \
        rng.normal(0, 0.1, [4, 64, 128]).astype(np.float32)

    def g(k):
        x0, x1, x3 = k.load(a), k.load(b), k.load(c)
        x6 = k.select(k.greater(x0, x1), k.add(x0, x3), k.mul(x1, x3))
        return [(k.store(k.add(x6, x0)), np.where(a > b, a + c, b * c) + a, None)]
    run_graph("eager", g)


def test_zero_sized_tensors():  # :674-725
    t = Tester("eager")
    out1 = t.store(t.mul(t.load(np.full([10, 0, 2], 0.1, np.float32)), 0.1))
    t.store_expect(t.mul(t.load(np.full([10, 1, 2], 0.2, np.float32)), 0.2), 0.2 * 0.2)
    assert t.run_check()
    assert out1.shape() == (10, 0, 2)
    t = Tester("eager")
    x3 = t.sum(t.add(t.load(np.full([10, 0, 2], 0.01, np.float32)), 0.1), (2,), True)
    out = t.store(t.sum(t.add(x3, 0.2), (1,), True))
    t.run()
    assert out.shape() == (10, 1, 1)
    assert np.array_equal(t.output(out), np.zeros([10, 1, 1], np.float32))
    t = Tester("eager")
    x2 = t.matmul(t.add(t.load(np.full([0, 1024], 0.001, np.float16)), 0.01), t.load(np.full([1024, 1024], 0.001, np.float16)), False, False)
    out = t.store(t.add(x2, 1.0))
    t.run()
    assert out.shape() == (0, 1024)


def test_small_graphs():  # :728-755
    a = np.random.default_rng(18).normal(0, 0.1, [10, 1024]).astype(np.float32)
    x1_e = a + 0.01
    x2_e = x1_e * x1_e

    def g(k):
        x1 = k.add(k.load(a), 0.01)
        x2 = k.mul(x1, x1)
        return [(k.store(k.add(k.add(x2, x2), x1)), (x2_e + x2_e) + x1_e, None)]
    run_graph("eager", g)
    run_graph("eager", lambda k: [(k.store(k.add(k.full(0.1, [256], "float32"), 0.2)), np.float32(0.3), None),
                                  (k.store(k.full(0.4, [512], "float32")), np.float32(0.4), None)])


def test_broadcast_reduce_reuse():  # :758-773
    rng = np.random.default_rng(19)
    a, b = rng.normal(0, 0.1, [1, 2000]).astype(np.float32), rng.normal(0, 0.1, [10, 2000]).astype(np.float32)
    e4 = np.sum(a * b, axis=(0,), keepdims=True)

    def g(k):
        x2 = k.load(b)
        x4 = k.sum(k.mul(k.load(a), x2), (0,), True)
        return [(k.store(k.sum(k.add(x4, x2), (0,), True)), np.sum(e4 + b, axis=(0,), keepdims=True), 1e-4)]
    run_graph("eager", g)


def test_broadcast_store_reuse():  # :775-791
    rng = np.random.default_rng(20)
    a0, a1 = rng.normal(-1, 1, [3000]).astype(np.float32), rng.normal(-1, 1, [10, 3000]).astype(np.float32)
    e1 = (a0 + 0.01) * 0.8

    def g(k):
        x1 = k.add(k.load(a0), 0.01)
        x2 = k.sum(x1, (0,), True)
        y1 = k.mul(x1, 0.8)
        y2 = k.add(y1, k.load(a1))
        return [(k.store(x2), np.sum(a0 + 0.01, axis=(0,), keepdims=True), 1e-4), (k.store(y2), e1 + a1, None), (k.store(y1), e1, None)]
    run_graph("eager", g)


@pytest.mark.parametrize("mode", ["eager", "eager:lazy", "eager:lazy,unify_ws"])
def test_matmul_users(mode):  # :811-826 (two casts of one product), :829-842 (two epilogues), :845-858 (two products added)
    rng = np.random.default_rng(21)
    a, b = rng.normal(0, 0.01, [1024, 1024]).astype(np.float16), rng.normal(0, 0.01, [1024, 512]).astype(np.float16)
    c, d = rng.normal(0, 0.01, [1024, 768]).astype(np.float16), rng.normal(0, 0.01, [768, 512]).astype(np.float16)
    e32 = np.matmul(a.astype(np.float32), b.astype(np.float32))
    e16 = e32.astype(np.float16)

    def g0(k):
        x2 = k.matmul(k.load(a), k.load(b), False, False)
        return [(k.store(k.add(k.cast(x2, "float32"), k.cast(x2, "float32"))), e32 + e32, 1e-3)]
    # the fp16 rounding of a product can fall either way when the fp32 sums differ in their last bit: one fp16 step
    run_graph(mode, g0, oracle_eps=1e-3)

    def g1(k):
        x2 = k.matmul(k.load(a), k.load(b), False, False)
        s3 = k.store(k.add(x2, 0.1))
        return [(s3, e16 + np.float16(0.1), 1e-3), (k.store(k.mul(x2, 0.5)), e16 * np.float16(0.5), 1e-3)]
    run_graph(mode, g1)

    def g2(k):
        x0 = k.matmul(k.load(a), k.load(b), False, False)
        x1 = k.matmul(k.load(c), k.load(d), False, False)
        return [(k.store(k.add(x0, x1)), e32 + np.matmul(c.astype(np.float32), d.astype(np.float32)), 1e-3)]
    run_graph(mode, g2)


@pytest.mark.parametrize("shape_a,shape_b,shape_c", [([1024, 512], [512, 256], [256, 1024]), ([4096, 640], [640, 8], [8, 640])])
def test_matmul_chain(shape_a, shape_b, shape_c):  # :861-876
    rng = np.random.default_rng(shape_a[0])
    a, b, c = (rng.normal(0, 0.01, s).astype(np.float16) for s in (shape_a, shape_b, shape_c))
    e0 = np.matmul(a.astype(np.float32), b.astype(np.float32))

    def g(k):
        x0 = k.matmul(k.load(a), k.load(b), False, False)
        return [(k.store(k.matmul(x0, k.load(c), False, False)), np.matmul(e0, c.astype(np.float32)).astype(np.float16), 1e-3)]
    run_graph("eager", g)


def test_reshape_between_areas():  # :879-903
    rng = np.random.default_rng(22)
    a0 = rng.normal(-1, 1, [600, 512]).astype(np.float16)
    run_graph("eager", lambda k: [(k.store(k.mul(k.reshape(k.add(k.load(a0), 0.01), [100, 48, 64]), 0.8)),
                                   np.reshape(a0 + np.float16(0.01), [100, 48, 64]) * np.float16(0.8), None)])
    a1 = rng.normal(-1, 1, [1, 60, 512]).astype(np.float16)
    e1 = a1 + np.float16(0.01)

    def g(k):
        x1 = k.add(k.load(a1), 0.01)
        x2 = k.reshape(x1, [60, 1, 512])
        x3 = k.mul(x2, x1)
        return [(k.store(x2), np.reshape(e1, [60, 1, 512]), None), (k.store(x3), np.reshape(e1, [60, 1, 512]) * e1, None)]
    run_graph("eager", g)


def test_lazy_unified_workspace():  # :906-917
    a = np.random.default_rng(23).normal(-0.5, 0.5, [30, 4000]).astype(np.float32)
    Tester.set_deterministic(True)
    try:
        run_graph("eager:unify_ws,lazy", lambda k: [(k.store(k.add(k.sum(k.mul(k.load(a), 1.5), (0,), True), 0.1)),
                                                     np.sum(a * np.float32(1.5), (0,), keepdims=True) + 0.1, None)])
    finally:
        Tester.set_deterministic(False)


def test_product_plus_a_strided_view():  # :793-806: the epilogue reads a [1024, 512] window of a [1024, 1000] buffer
    rng = np.random.default_rng(793)
    a = rng.normal(0, 0.01, [1024, 1024]).astype(np.float16)
    b = rng.normal(0, 0.01, [1024, 512]).astype(np.float16)
    c = rng.normal(0, 1, [1024, 1000]).astype(np.float16)
    t = Tester("eager")
    x2 = t.matmul(t.load(a), t.load(b), False, False)
    x4 = t.add(x2, t.view_load([1024, 512], [1000, 1], c))
    t.store_expect(x4, np.matmul(a.astype(np.float32), b.astype(np.float32)).astype(np.float16) + c[:, :512])
    assert t.run_check()
    assert t.das().count("mmad acc, A, B") == 1 and "Add.fp16 acc, m" in t.das(), t.das()  # the add rides in the matmul's epilogue


def test_lazy_tuning_switch_is_accepted():  # :371-385: the same product three times on one kernel object, tuner on
    rng = np.random.default_rng(371)
    a = rng.normal(0, 0.01, [4096, 4096]).astype(np.float16)
    b = rng.normal(0, 0.01, [4096, 4096]).astype(np.float16)
    expect = np.matmul(a.astype(np.float32), b.astype(np.float32))
    t = Tester("eager")
    Tester.set_lazy_tuning(True)
    try:
        for _ in range(3):
            t.store_expect(t.matmul(t.load(a), t.load(b), False, False), expect, 1e-3)
            assert t.run_check()
            t.reset()
    finally:
        Tester.set_lazy_tuning(False)
