"""GPU parity: reshape between operators, restating tests/ut/test_reshape.py of the reference (cited per test):
same shapes, inputs, NumPy expectations and tolerances, default kernel type as there; every graph also runs on
the CPU oracle. A reshape of a computed value is a view of its buffer here: the value is written once and read
back through the new shape, which is what these graphs probe (which launch writes, which reads, in what shape)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dims", [(2,), (1,)])
def test_reduce_forward(dims):  # tests/ut/test_reshape.py:20-38
    b = np.full((10, 3, 1), 0.1, np.float32)
    e = np.sum(np.reshape(np.broadcast_to(b, (10, 3, 4)), (1, 10, 12)), dims, keepdims=True)
    run_graph("", lambda k: [(k.store(k.sum(k.reshape(k.broadcast(k.load(b), (10, 3, 4)), (1, 10, 12)), dims, True)), e, None)])


def test_unary_and_cast():  # :41-70
    x = np.full((16, 16), 81.0, np.float32)
    run_graph("", lambda k: [(k.store(k.sqrt(k.reshape(k.sqrt(k.load(x)), (32, 8)))), np.float32(3.0), None)])
    run_graph("", lambda k: [(k.store(k.cast(k.sqrt(k.reshape(k.sqrt(k.load(x)), (32, 8))), "float16")), np.float16(3.0), None)])


def test_select_forward():  # :73-90
    a, b = np.full((9,), 1.0, np.float32), np.full((3, 3), 2.0, np.float32)
    c = np.random.default_rng(1).choice([True, False], (3, 3)).astype(bool)
    run_graph("", lambda k: [(k.store(k.select(k.load(c), k.reshape(k.load(a), (3, 3)), k.load(b))), np.where(c, a.reshape(3, 3), b), 1e-5)])


def test_broadcasts_around_reshape():  # :93-128
    b = np.full([1, 8], 0.3, np.float32)
    run_graph("", lambda k: [(k.store(k.broadcast(k.reshape(k.broadcast(k.load(b), [10, 8]), [10, 1, 8]), [10, 4, 8])), np.float32(0.3), None)])
    c = np.full([10, 3, 4], 0.3, np.float32)
    run_graph("", lambda k: [(k.store(k.broadcast(k.reshape(k.load(c), [1, 10, 12]), [8, 10, 12])), np.float32(0.3), None)])
    run_graph("", lambda k: [(k.store(k.broadcast(k.reshape(k.full(0.3, [3, 10], "float32"), [3, 1, 10]), [3, 10, 10])), np.float32(0.3), None)])


def test_multi_reshape():  # :131-158
    a = np.random.default_rng(2).random((54, 89)).astype(np.float32) + np.float32(0.01)

    def g1(k):
        x = k.load(a)
        return [(k.store(k.add(k.sqrt(k.reshape(x, [89, 54])), k.reshape(k.reciprocal(x), [89, 54]))),
                 np.add(np.sqrt(a), np.reciprocal(a)).reshape([89, 54]), None)]
    run_graph("", g1)
    run_graph("", lambda k: [(k.store(k.reshape(k.sqrt(k.reshape(k.load(a), [89, 54])), [178, 27])), np.sqrt(a).reshape([178, 27]), None)])


def test_unalign_broadcast():  # :176-189
    a, b = np.full([1, 320], 0.3, np.float16), np.full((), 0.2, np.float32)
    run_graph("", lambda k: [(k.store(k.mul(k.reshape(k.cast(k.load(a), "float32"), [320]), k.load(b))), np.float32(0.06), 1e-3)])


@pytest.mark.parametrize("shape1,shape2,shape3", [([10, 20, 8], [20, 8], [200, 8]), ([10, 20, 8], [8], [200, 8]), ([10, 20, 8], [8], [10, 160])])
def test_unalign_broadcast_2(shape1, shape2, shape3):  # :192-208
    a, b = np.full(shape1, 0.3, np.float32), np.full(shape2, 0.2, np.float32)
    run_graph("", lambda k: [(k.store(k.mul(k.reshape(k.add(k.load(a), k.load(b)), shape3), 0.1)), np.float32(0.05), None)])


def test_reduce_lead_dim():  # :211-220
    a = np.random.default_rng(3).normal(-0.5, 0.5, [128, 1]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.sum(k.reshape(k.load(a), [1, 128]), [1], True)), np.sum(a, (0,), keepdims=True), None)])


@pytest.mark.parametrize("shape1,shape2", [([2, 3, 64], [2, 6, 32]), ([1000, 4], [100, 40]), ([128], [128, 1])])
def test_reshape_then_op_or_store(shape1, shape2):  # :223-248
    a = np.full(shape1, 0.3, np.float32)
    run_graph("", lambda k: [(k.store(k.sqrt(k.reshape(k.mul(k.load(a), 0.6), shape2))), np.float32(0.42426), 1e-5)])
    run_graph("", lambda k: [(k.store(k.reshape(k.mul(k.load(a), 0.6), shape2)), np.float32(0.18), None)])


@pytest.mark.parametrize("shape1,shape2", [([1000, 4], [100, 40]), ([1000, 4], [20, 5, 40]), ([3, 1000, 4], [3, 20, 5, 40]),
                                           ([3, 20, 5, 4, 2], [3, 10, 40, 2]), ([3, 2, 10, 64], [6, 10, 16, 4]),
                                           ([3, 2, 1, 10], [6, 1, 10]), ([3, 2, 1, 1, 10], [6, 1, 10]), ([3, 2, 1, 10], [6, 1, 1, 10])])
def test_reshape_shapes(shape1, shape2):  # :251-270
    a = np.random.default_rng(len(shape1) * 10 + len(shape2)).normal(0.0, 1.0, shape1).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.reshape(k.mul(k.load(a), 0.6), shape2), 0.1)),
                              (a * np.float32(0.6)).reshape(shape2) + np.float32(0.1), None)])


@pytest.mark.parametrize("shape_a,shape_b,shape_c,red", [([10, 64], [10, 1], [2, 5, 64], (1,)), ([10, 64], [10, 1], [10, 4, 16], (2,)),
                                                         ([10, 4, 64], [10, 4, 1], [10, 32, 8], (0,)), ([2, 10, 64], [64], [20, 64], (1,)),
                                                         ([10, 4, 64], [10, 4, 1], [10, 32, 8], (1,))])
def test_add_reshape_reduce(shape_a, shape_b, shape_c, red):  # :273-293
    rng = np.random.default_rng(shape_c[-1] + red[0])
    a, b = rng.normal(0.0, 0.3, shape_a).astype(np.float32), rng.normal(0.0, 0.2, shape_b).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.sum(k.reshape(k.add(k.load(a), k.load(b)), shape_c), red, True)),
                              np.sum((a + b).reshape(shape_c), axis=red, keepdims=True), 1e-4)])


def test_matmul_then_reshape():  # :296-311
    np.random.seed(4)
    ax = Tester.fast_random_normal(0, 0.01, [1020, 3072]).astype(np.float16)
    bx = Tester.fast_random_normal(0, 0.01, [3072, 3072]).astype(np.float16)
    e = np.matmul(ax.astype(np.float32), bx.astype(np.float32)).astype(np.float16)
    run_graph("mix", lambda k: [(k.store(k.reshape(k.matmul(k.load(ax), k.load(bx), False, False), (2, 510, 48, 64))),
                                 np.reshape(e, (2, 510, 48, 64)), 2e-3)], oracle=False)  # 9.6 GFLOP: NumPy golden only


@pytest.mark.parametrize("shape_a,shape_b,shape_c", [([1, 8, 2048, 512], [1, 8, 512, 128], [8, 2048, 128]), ([2048, 512], [512, 512], [2048, 1, 512]),
                                                     ([2048, 512], [512, 512], [1024, 1024]), ([2048, 512], [512, 512], [1, 2048, 512, 1, 1]),
                                                     ([2048, 512], [512, 512], [2048 * 512])])
def test_matmul_reshape_add(shape_a, shape_b, shape_c):  # :314-334
    np.random.seed(5)
    ax, bx, cx = (Tester.fast_random_normal(0, 0.01, s).astype(np.float16) for s in (shape_a, shape_b, shape_c))
    e = np.matmul(ax.astype(np.float32), bx.astype(np.float32)).astype(np.float16)
    run_graph("mix", lambda k: [(k.store(k.add(k.reshape(k.matmul(k.load(ax), k.load(bx), False, False), shape_c), k.load(cx))),
                                 np.reshape(e, shape_c) + cx, 2e-3)], oracle_eps=2e-3)


@pytest.mark.parametrize("shape_c", [[512, 1, 768], [4, 128, 768]])
def test_matmul_reshape_broadcast_add(shape_c):  # :337-352
    np.random.seed(6)
    ax, bx, dx = (Tester.fast_random_normal(0, 0.01, s).astype(np.float16) for s in ([512, 1024], [1024, 768], [768]))
    e = np.reshape(np.matmul(ax.astype(np.float32), bx.astype(np.float32)).astype(np.float16), shape_c) + dx
    run_graph("mix", lambda k: [(k.store(k.add(k.reshape(k.matmul(k.load(ax), k.load(bx), False, False), shape_c), k.load(dx))), e, 2e-3)],
              oracle_eps=2e-3)


def test_reshape_of_loads():  # :355-378
    rng = np.random.default_rng(7)
    a, b = rng.normal(-0.5, 0.5, [128]).astype(np.float32), rng.normal(-0.5, 0.5, [100, 128]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.reshape(k.load(a), [1, 128]), k.load(b))), np.reshape(a, [1, 128]) + b, None)])
    bf = b.reshape(100 * 128)
    run_graph("", lambda k: [(k.store(k.mul(k.reshape(k.load(a), [1, 128]), k.reshape(k.load(bf), [100, 128]))), np.reshape(a, [1, 128]) * b, None)])


def test_two_views_of_one_load():  # :381-395, :412-421
    rng = np.random.default_rng(8)
    a, b = rng.normal(-0.5, 0.5, [4, 1, 1, 512]).astype(np.float32), rng.normal(-0.5, 0.5, [4, 64, 512]).astype(np.float32)

    def g(k):
        x1 = k.add(k.load(a), 0.01)
        x2 = k.load(b)
        x5 = k.add(k.reshape(x2, [4, 64, 1, 512]), k.reshape(x2, [4, 1, 64, 512]))
        return [(k.store(k.mul(x1, x5)), (a + np.float32(0.01)) * (np.reshape(b, [4, 64, 1, 512]) + np.reshape(b, [4, 1, 64, 512])), None)]
    run_graph("", g)
    c = rng.normal(0.0, 0.03, [10, 1000]).astype(np.float32)

    def g2(k):
        x0 = k.load(c)
        return [(k.store(k.add(k.reshape(x0, [1, 10, 1000]), k.reshape(x0, [10, 1, 1000]))), c.reshape([1, 10, 1000]) + c.reshape([10, 1, 1000]), None)]
    run_graph("", g2)


def test_value_and_its_reshape_meet_again():  # :398-409, :436-452
    rng = np.random.default_rng(9)
    a = rng.normal(0.0, 0.03, [10, 1, 1000]).astype(np.float32)

    def g(k):
        x1 = k.add(k.load(a), 0.1)
        return [(k.store(k.mul(k.reshape(x1, [1, 10, 1000]), x1)), (a + np.float32(0.1)).reshape([1, 10, 1000]) * (a + np.float32(0.1)), None)]
    run_graph("", g)
    b = rng.normal(0.0, 0.3, [8, 1]).astype(np.float32)

    def g2(k):
        x0 = k.load(b)
        x4 = k.reshape(k.broadcast(k.reshape(k.broadcast(x0, [8, 16]), [8, 16, 1]), [8, 16, 32]), [8, 512])
        return [(k.store(k.add(x4, k.broadcast(k.mul(x0, 0.1), [8, 512]))),
                 np.broadcast_to(b, [8, 512]) + np.broadcast_to(b * np.float32(0.1), [8, 512]), None)]
    run_graph("", g2)


def test_reshape_expand_outmost_dim():  # :424-433
    rng = np.random.default_rng(10)
    a, b = rng.normal(0.0, 0.01, [1, 10, 1, 200]).astype(np.float32), rng.normal(0.0, 0.01, [10, 20, 200]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.reshape(k.load(a), [10, 1, 200]), k.load(b))), a.reshape([10, 1, 200]) + b, None)])
