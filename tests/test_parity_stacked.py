"""GPU parity: sequence ("seq") and parallel kernels, whose sub-kernel groups the caller marks.

Each case restates a case of the reference's tests/ut/test_sequence_fusion.py or
test_parallel_fusion.py (cited per test): same shapes, input distributions, NumPy golden and
tolerance. The same graph also runs on the CPU oracle, and the two must agree to the usual bar
(fp32 1e-5, fp16 1e-3, bf16 1e-2)."""
import numpy as np
import pytest

from dvm_amd import DataType
from dvm_amd.tester import Tester
from oracle.oracle import OracleKernel

pytestmark = pytest.mark.gpu

EPS = {int(DataType.float32): 1e-5, int(DataType.float16): 1e-3, int(DataType.bfloat16): 1e-2}


def run_both(ker, build, goldens, eps=None, oracle_eps=None, min_launches=None):
    """build(k) -> list of stores. Runs on the HIP path and on the oracle, compares both and the goldens."""
    t = Tester(ker)
    stores = build(t)
    o = OracleKernel()
    refs = [o.output(v) for v in build(o)]
    t.run()
    if min_launches is not None:
        assert t.num_launches() >= min_launches, t.das()
    for i, (s, ref, gold) in enumerate(zip(stores, refs, goldens)):
        out = t.output(s)
        dt = int(s.dtype())
        if dt == int(DataType.bfloat16):
            out = Tester.convert_from_bf16(out)
        e = oracle_eps if oracle_eps is not None else EPS[dt]
        assert np.allclose(out.astype(np.float32), ref.astype(np.float32), rtol=e, atol=e), (
            "output %d differs from the oracle: max abs diff %g\n%s"
            % (i, np.abs(out.astype(np.float64) - ref.astype(np.float64)).max(), t.das()))
        if gold is not None:
            g = eps if eps is not None else EPS[dt]
            assert np.allclose(out, gold, rtol=g, atol=g), "output %d differs from the NumPy golden" % i
    return t


def test_seq_vec_vec():  # tests/ut/test_sequence_fusion.py:22-33
    ax = np.full([1024, 128], 0.05, np.float32)

    def g(k):
        k.seq_add(k.K_VEC)
        a = k.load(ax)
        c = k.mul(a, k.add(a, 0.2))
        k.seq_add(k.K_VEC)
        return [k.store(k.mul(c, 0.7))]
    run_both("seq", g, [(ax + 0.2) * ax * 0.7], min_launches=2)


def test_seq_vec_mix():  # tests/ut/test_sequence_fusion.py:38-53
    rng = np.random.default_rng(1)
    ax = rng.normal(0, 1, [1024, 512]).astype(np.float16)
    fx = rng.normal(0, 1, [512, 1024]).astype(np.float16)

    def g(k):
        k.seq_add(k.K_VEC)
        a = k.load(ax)
        c = k.mul(a, k.add(a, 0.02))
        k.seq_add(k.K_MIX)
        return [k.store(k.cast(k.matmul(c, k.load(fx), False, False), "float32"))]
    # the reference checks against fp32 NumPy at 1e-3 with fp16-rounded products of N(0,1) inputs in
    # the hundreds; relative to the output scale that is what the golden tolerance below states
    c16 = ((ax + np.float16(0.02)) * ax)
    gold = np.matmul(c16.astype(np.float32), fx.astype(np.float32))
    t = Tester("seq")
    st = g(t)
    o = OracleKernel()
    ref = o.output(g(o)[0])
    t.run()
    out = t.output(st[0])
    assert t.num_launches() == 2
    assert np.allclose(out, ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max())
    assert np.allclose(out, gold, rtol=2e-3, atol=2e-3 * np.abs(gold).max())


def test_seq_mix_vec():  # tests/ut/test_sequence_fusion.py:58-73
    rng = np.random.default_rng(2)
    ax = rng.normal(0, 1, [768, 512]).astype(np.float16)
    bx = rng.normal(0, 1, [512, 128 * 7]).astype(np.float16)

    def g(k):
        k.seq_add(k.K_MIX)
        d = k.cast(k.matmul(k.load(ax), k.load(bx), False, False), "float32")
        k.seq_add(k.K_VEC)
        return [k.store(k.add(d, 0.02))]
    gold = np.matmul(ax.astype(np.float32), bx.astype(np.float32)).astype(np.float16).astype(np.float32) + 0.02
    t = Tester("seq")
    st = g(t)
    o = OracleKernel()
    ref = o.output(g(o)[0])
    t.run()
    out = t.output(st[0])
    assert t.num_launches() == 2
    assert np.allclose(out, ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max())
    assert np.allclose(out, gold, rtol=2e-3, atol=2e-3 * np.abs(gold).max())


def test_seq_inplace_reuse():  # tests/ut/test_sequence_fusion.py:78-90
    ax = np.full([1024], 0.05, np.float32)

    def g(k):
        k.seq_add(k.K_VEC)
        a1 = k.add(k.load(ax), 0.1)
        k.seq_add(k.K_VEC)
        b1 = k.add(a1, 0.1)
        k.seq_add(k.K_VEC)
        return [k.store(k.add(b1, 0.1))]
    run_both("seq", g, [np.full([1024], 0.05 + 0.3, np.float32)], min_launches=3)


def test_seq_inplace_stage():  # tests/ut/test_sequence_fusion.py:95-114
    ax = np.full([1024], 0.05, np.float32)

    def g(k):
        k.seq_add(k.K_VEC)
        a1 = k.cast(k.load(ax), "float16")
        k.seq_add(k.K_VEC)
        b1 = k.cast(a1, "float32")
        k.seq_add(k.K_VEC)
        c1 = k.cast(b1, "float16")
        k.seq_add(k.K_VEC)
        d1 = k.add(c1, 0.1)
        k.seq_add(k.K_VEC)
        e1 = k.add(d1, 0.1)
        k.seq_add(k.K_VEC)
        return [k.store(k.cast(e1, "float32"))]
    run_both("seq", g, [np.full([1024], 0.05 + 0.2, np.float32)], eps=1e-3, min_launches=6)


def test_seq_inplace_multi():  # tests/ut/test_sequence_fusion.py:119-131
    ax = np.full([1024], 0.05, np.float32)

    def g(k):
        k.seq_add(k.K_VEC)
        a0 = k.load(ax)
        a1, a2 = k.add(a0, 0.1), k.mul(a0, 0.5)
        k.seq_add(k.K_VEC)
        return [k.store(k.add(k.div(a1, 0.8), a2))]
    run_both("seq", g, [np.divide(ax + 0.1, 0.8) + ax * 0.5], min_launches=2)


def test_seq_workspace_reuse():  # tests/ut/test_sequence_fusion.py:136-152
    rng = np.random.default_rng(3)
    ax = rng.normal(0, 1, [512, 512]).astype(np.float16)
    bx = rng.normal(0, 1, [512, 512]).astype(np.float16)

    def g(k):
        k.seq_add(k.K_MIX)
        d = k.cast(k.matmul(k.load(ax), k.load(bx), False, False), "float32")
        k.seq_add(k.K_VEC)
        f1 = k.cast(d, "float16")
        k.seq_add(k.K_VEC)
        return [k.store(k.cast(f1, "float32"))]
    gold = np.matmul(ax.astype(np.float32), bx.astype(np.float32))
    run_both("seq", g, [gold], eps=1e-2 * 25, oracle_eps=1e-3 * 25, min_launches=3)


def test_seq_extern_code():  # tests/ut/test_sequence_fusion.py:157-173: 400 operators behind a matmul
    rng = np.random.default_rng(4)
    ax = rng.normal(0, 1, [512, 512]).astype(np.float16)
    bx = rng.normal(0, 1, [512, 512]).astype(np.float16)

    def g(k):
        k.seq_add(k.K_MIX)
        f = k.cast(k.matmul(k.load(ax), k.load(bx), False, False), "float32")
        k.seq_add(k.K_VEC)
        for _ in range(200):
            f = k.sub(k.add(f, 0.01), 0.01)
        return [k.store(f)]
    gold = np.matmul(ax.astype(np.float32), bx.astype(np.float32))
    run_both("seq", g, [gold], eps=1e-2 * 25, oracle_eps=1e-3, min_launches=2)


def test_seq_vec_reduce():  # tests/ut/test_sequence_fusion.py:178-209: RMSNorm in three groups, stores read back
    rng = np.random.default_rng(1)
    a0 = Tester.bf16_random_normal(-1, 1, [1, 2048, 5120])
    a1 = rng.normal(-1, 1, [5120]).astype(np.float32)
    e5 = 1.0 / np.sqrt(np.sum(a0 * a0, (2,), keepdims=True) * 0.000195313 + 1e-6)
    e7 = a0 * e5 * a1

    def g(k):
        k.seq_add(k.K_VEC)
        y0 = k.cast(k.load(a0, "bfloat16"), "float32")
        o0 = k.store(y0)
        y2 = k.sum(k.mul(y0, y0), (2,), True)
        k.seq_add(k.K_VEC)
        y5 = k.reciprocal(k.sqrt(k.add(k.mul(y2, 0.000195313), 1e-6)))
        o5 = k.store(y5)
        k.seq_add(k.K_VEC)
        y7 = k.mul(k.mul(o0, o5), k.load(a1))
        return [o0, o5, k.store(k.cast(y7, "bfloat16"))]
    run_both("seq", g, [a0, e5, e7], eps=1e-2, min_launches=3)


def test_seq_broadcast_store_reuse():  # tests/ut/test_sequence_fusion.py:214-229
    rng = np.random.default_rng(5)
    a0 = rng.normal(-1, 1, [3000]).astype(np.float32)
    a1 = rng.normal(-1, 1, [10, 3000]).astype(np.float32)

    def g(k):
        k.seq_add(k.K_VEC)
        x1 = k.add(k.load(a0), 0.01)
        k.seq_add(k.K_VEC)
        y1 = k.mul(x1, 0.8)
        y2 = k.add(y1, k.load(a1))
        return [k.store(y1), k.store(y2)]
    e1 = (a0 + 0.01) * 0.8
    run_both("seq", g, [e1, e1 + a1], min_launches=2)


def test_seq_reloc_depend():  # tests/ut/test_sequence_fusion.py:234-249
    rng = np.random.default_rng(6)
    a0 = rng.normal(-1, 1, [3, 18911]).astype(np.float32)
    a1 = rng.normal(-1, 1, [3, 1]).astype(np.float32)

    def g(k):
        k.seq_add(k.K_VEC)
        x1 = k.add(k.load(a0), 0.01)
        k.seq_add(k.K_VEC)
        y1 = k.mul(x1, 0.8)
        y2 = k.add(y1, k.load(a1))
        return [k.store(y1), k.store(y2)]
    e1 = (a0 + 0.01) * 0.8
    run_both("seq", g, [e1, e1 + a1], min_launches=2)


def test_seq_vec_mix_dyn():  # tests/ut/test_sequence_fusion.py:254-275: shapes change between runs
    t = Tester("seq:dyn")
    t.seq_add(Tester.K_VEC)
    x0 = t.load([-1], "float16")
    x2 = t.mul(t.add(x0, 0.02), x0)
    t.seq_add(Tester.K_MIX)
    y0 = t.load([-1], "float16")
    y2 = t.cast(t.matmul(x2, y0, False, False), "float32")
    t.seq_add(Tester.K_VEC)
    out = t.store(t.sub(y2, 0.01))
    rng = np.random.default_rng(7)
    for xs, ys in [[[512, 1024], [1024, 512]], [[768, 1024], [1024, 1024]]]:
        xd = rng.normal(0, 1, xs).astype(np.float16)
        yd = rng.normal(0, 1, ys).astype(np.float16)
        t.input(x0, xd)
        t.input(y0, yd)
        t.run()
        got = t.output(out)
        c16 = (xd + np.float16(0.02)) * xd
        gold = np.matmul(c16.astype(np.float32), yd.astype(np.float32)).astype(np.float16).astype(np.float32) - 0.01
        assert got.shape == gold.shape
        assert np.allclose(got, gold, rtol=2e-3, atol=2e-3 * np.abs(gold).max())


@pytest.mark.parametrize("shapes", [([256], [256], [1024]), ([8192 * 2], [8192 * 4], [4096])])
def test_parallel_basic(shapes):  # tests/ut/test_parallel_fusion.py:26-48
    def g(k):
        k.parallel_add(k.K_VEC)
        s0 = k.store(k.mul(k.load(np.full(shapes[0], 0.1, np.float32)), 0.3))
        k.parallel_add(k.K_VEC)
        s1 = k.store(k.add(k.load(np.full(shapes[1], 0.1, np.float32)), 0.3))
        k.parallel_add(k.K_VEC)
        s2 = k.store(k.add(k.load(np.full(shapes[2], 0.1, np.float32)), 0.3))
        return [s0, s1, s2]
    run_both("parallel", g, [np.full(shapes[0], 0.1 * 0.3, np.float32), np.full(shapes[1], 0.4, np.float32),
                             np.full(shapes[2], 0.4, np.float32)], min_launches=3)


@pytest.mark.parametrize("determ", [False, True])
def test_parallel_reduce(determ):  # tests/ut/test_parallel_fusion.py:52-90; reductions here have one fixed order
    def g(k):
        k.parallel_add(k.K_VEC)
        s0 = k.store(k.sum(k.load(np.full((8192,), 0.1, np.float32)), [0], False))
        k.parallel_add(k.K_VEC)
        s1 = k.store(k.sum(k.load(np.full((4, 4096), 0.1, np.float32)), [0], False))
        k.parallel_add(k.K_VEC)
        s2 = k.store(k.add(k.load(np.full((1,), 0.1, np.float32)), 1.0))
        return [s0, s1, s2]
    Tester.set_deterministic(determ)
    try:
        run_both("parallel", g, [np.float32(8192 * 0.1), np.full((4096,), 0.4, np.float32),
                                 np.full((1,), 1.1, np.float32)], min_launches=3)
    finally:
        Tester.set_deterministic(False)


def _mm_f16(a, b):
    return np.matmul(a.astype(np.float32), b.astype(np.float32)).astype(np.float16)


@pytest.mark.parametrize("k1, k2", [(Tester.K_CUBE, Tester.K_CUBE), (Tester.K_CUBE, Tester.K_MIX),
                                    (Tester.K_MIX, Tester.K_MIX)])
def test_parallel_cube_cube(k1, k2):  # tests/ut/test_parallel_fusion.py:93-121
    np.random.seed(21)
    xa = Tester.fast_random_normal(0, 0.1, [1024, 768]).astype(np.float16)
    xb = Tester.fast_random_normal(0, 0.1, [768, 2000]).astype(np.float16)
    ya = Tester.fast_random_normal(0, 0.1, [500, 1024]).astype(np.float16)
    yb = Tester.fast_random_normal(0, 0.1, [1024, 1600]).astype(np.float16)

    def g(k):
        k.parallel_add(k1)
        x2 = k.matmul(k.load(xa), k.load(xb), False, False)
        if k1 == Tester.K_MIX:
            x2 = k.mul(x2, 0.5)
        s0 = k.store(x2)
        k.parallel_add(k2)
        y2 = k.matmul(k.load(ya), k.load(yb), False, False)
        if k2 == Tester.K_MIX:
            y2 = k.add(y2, 0.3)
        return [s0, k.store(y2)]
    x_e, y_e = _mm_f16(xa, xb), _mm_f16(ya, yb)
    run_both("parallel", g, [x_e * 0.5 if k1 == Tester.K_MIX else x_e, y_e + 0.3 if k2 == Tester.K_MIX else y_e],
             eps=1e-3, min_launches=2)


@pytest.mark.parametrize("ktype", [Tester.K_CUBE, Tester.K_MIX])
def test_parallel_cube_vector(ktype):  # tests/ut/test_parallel_fusion.py:124-146
    np.random.seed(22)
    xa = Tester.fast_random_normal(0, 0.1, [1024, 768]).astype(np.float16)
    xb = Tester.fast_random_normal(0, 0.1, [768, 2000]).astype(np.float16)
    ya = np.random.normal(0, 0.1, [10, 1024]).astype(np.float16)

    def g(k):
        k.parallel_add(ktype)
        x2 = k.matmul(k.load(xa), k.load(xb), False, False)
        if ktype == Tester.K_MIX:
            x2 = k.mul(x2, 0.5)
        s0 = k.store(x2)
        k.parallel_add(k.K_VEC)
        y0 = k.load(ya)
        return [s0, k.store(k.cast(k.mul(k.add(y0, 0.3), y0), "float32"))]
    x_e = _mm_f16(xa, xb)
    run_both("parallel", g, [x_e * 0.5 if ktype == Tester.K_MIX else x_e, ((ya + 0.3) * ya).astype(np.float32)],
             eps=1e-3, oracle_eps=1e-3, min_launches=2)


@pytest.mark.parametrize("limits", [(0, 0, 0), (8, 8, 0), (0, 0, 10)])
def test_parallel_mix_cube_vector(limits):  # tests/ut/test_parallel_fusion.py:150-170: core limits are advice
    np.random.seed(23)
    xa = Tester.fast_random_normal(0, 0.1, [1024, 768]).astype(np.float16)
    xb = Tester.fast_random_normal(0, 0.1, [768, 2000]).astype(np.float16)
    ya = Tester.fast_random_normal(0, 0.1, [1536, 768]).astype(np.float16)
    yb = Tester.fast_random_normal(0, 0.1, [768, 768]).astype(np.float16)
    za = np.random.normal(0, 0.1, [10, 2000]).astype(np.float32)

    def g(k):
        k.parallel_add(k.K_MIX, 0, limits[0])
        s0 = k.store(k.mul(k.matmul(k.load(xa), k.load(xb), False, False), 0.5))
        k.parallel_add(k.K_CUBE, 0, limits[1])
        s1 = k.store(k.matmul(k.load(ya), k.load(yb), False, False))
        k.parallel_add(k.K_VEC, 0, limits[2])
        return [s0, s1, k.store(k.sum(k.add(k.load(za), 0.3), (0,), True))]
    run_both("parallel", g, [_mm_f16(xa, xb) * 0.5, _mm_f16(ya, yb), np.sum(za + 0.3, (0,), keepdims=True)],
             min_launches=3)


@pytest.mark.parametrize("ktype", [Tester.K_CUBE, Tester.K_MIX])
def test_parallel_cube_vector_dyn(ktype):  # tests/ut/test_parallel_fusion.py:174-220: ranks and shapes change per run
    t = Tester("parallel:dyn")
    t.parallel_add(ktype)
    xa, xb = t.load([-1], "float16"), t.load([-1], "float16")
    x0 = t.matmul(xa, xb, False, False)
    if ktype == Tester.K_MIX:
        x0 = t.add(t.mul(x0, 0.5), 0.02)
    x_out = t.store(x0)
    t.parallel_add(Tester.K_VEC)
    ya, yb = t.load([-1], "float32"), t.load([-1], "float32")
    y_out = t.store(t.sum(t.add(ya, yb), (1,), True))
    rng = np.random.default_rng(24)
    for sxa, sxb, sya, syb in [[[512, 2048], [2048, 1024], [1, 2000, 128], [4, 1, 128]],
                               [[2, 1024, 768], [768, 1024], [1, 512], [4000, 512]],
                               [[512, 1024], [1024, 768], [1024, 200], [1024, 200]]]:
        xad, xbd = rng.normal(0, 0.1, sxa).astype(np.float16), rng.normal(0, 0.1, sxb).astype(np.float16)
        yad, ybd = rng.normal(0, 0.1, sya).astype(np.float32), rng.normal(0, 0.1, syb).astype(np.float32)
        for h, d in ((xa, xad), (xb, xbd), (ya, yad), (yb, ybd)):
            t.input(h, d)
        t.run()
        x_e = _mm_f16(xad, xbd)
        if ktype == Tester.K_MIX:
            x_e = x_e * 0.5 + 0.02
        assert t.check(x_out, x_e, 1e-3)
        assert t.check(y_out, np.sum(yad + ybd, (1,), keepdims=True), 1e-3)
