"""GPU parity: the matmul cases of the reference's tests/ut/test_matmul.py beyond those in test_parity_matmul.py:
very wide N, folded batches (a unit axis between batch and k), one operand used twice, a single-row product
with a long k, the product + epilogue graphs written for other store paths (same mathematics here), dynamic
shapes run repeatedly. NumPy expectations and tolerances as in the reference; the oracle where it takes seconds."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def _close(out, want, eps):
    return np.allclose(out, want, rtol=eps, atol=eps)


def test_matmul_n_big():  # tests/ut/test_matmul.py:455-472
    np.random.seed(1)
    ax, bx = Tester.fast_random_normal(0, 0.1, [256, 256]).astype(np.float16), Tester.fast_random_normal(0, 0.1, [81960, 256]).astype(np.float16)
    np_c = np.matmul(ax.astype(np.float32), bx.astype(np.float32).T).astype(np.float16)
    zx = Tester.fast_random_normal(0, 0.1, np_c.shape).astype(np.float16)
    run_graph("mix", lambda k: [(k.store(k.add(k.matmul(k.load(ax), k.load(bx), False, True), k.load(zx))), np_c + zx, 2e-3)], oracle=False)


@pytest.mark.parametrize("shape_a,shape_b,shape_bias", [([256, 1, 1000], [1000, 256], None), ([256, 1, 1000], [1000, 256], [256, 1, 256]),
                                                        ([256, 1, 1000], [1000, 256], [1, 256]), ([520, 1, 40960], [40960, 256], [520, 1, 256]),
                                                        ([520, 1, 40960], [40960, 256], [1, 256])])
def test_batch_fold(shape_a, shape_b, shape_bias):  # :537-561
    np.random.seed(2)
    a, b = Tester.fast_random_normal(0, 0.1, shape_a).astype(np.float16), Tester.fast_random_normal(0, 0.1, shape_b).astype(np.float16)
    expect = np.matmul(a.astype(np.float32), b.astype(np.float32)).astype(np.float16)
    bias = Tester.fast_random_normal(0, 0.1, shape_bias).astype(np.float16) if shape_bias else None

    def g(k):
        out = k.matmul(k.load(a), k.load(b), False, False)
        if bias is not None:
            out = k.add(out, k.load(bias))
        return [(k.store(out), expect + bias if bias is not None else expect, 2e-3)]
    run_graph("mix", g, oracle=shape_a[-1] <= 1000, oracle_eps=2e-3)


def test_batch_fold_broadcast():  # :562-583
    np.random.seed(3)
    a0 = Tester.fast_random_normal(0, 0.1, [632, 1, 3584]).astype(np.float16)
    a1 = Tester.fast_random_normal(0, 0.1, [4608, 3584]).astype(np.float16)
    a4 = np.random.normal(0, 0.1, [4608]).astype(np.float16)
    e2 = np.matmul(a0.astype(np.float32), a1.swapaxes(-1, -2).astype(np.float32)).astype(np.float16)

    def g(k):
        x3 = k.cast(k.matmul(k.load(a0), k.load(a1), False, True), "float32")
        return [(k.store(k.cast(k.add(x3, k.cast(k.load(a4), "float32")), "float16")), (e2.astype(np.float32) + a4.astype(np.float32)).astype(np.float16), 1e-3)]
    run_graph("mix", g, oracle=False)


@pytest.mark.parametrize("shape_a,shape_b", [([256, 256], [256, 256]), ([1024, 128], [128, 1024]), ([301, 256], [256, 401]),
                                             ([300, 6400], [6400, 10240])])
@pytest.mark.parametrize("z32", [False, True])
def test_product_plus_tensor_abs(shape_a, shape_b, z32):  # :584-668 (three store paths there, one here)
    rng = np.random.default_rng(shape_a[0])
    ax, bx = rng.normal(0, 0.1, shape_a).astype(np.float16), rng.normal(0, 0.1, shape_b).astype(np.float16)
    np_c = np.matmul(ax.astype(np.float32), bx.astype(np.float32))
    zx = rng.normal(0, 0.1, np_c.shape).astype(np.float32 if z32 else np.float16)

    def g(k):
        c = k.matmul(k.load(ax), k.load(bx), False, False)
        if z32:
            c = k.cast(c, "float32")
        return [(k.store(k.abs(k.add(c, k.load(zx)))), np.abs(np_c + zx), 2e-3 * max(1.0, float(np.abs(np_c).max())))]
    run_graph("mix", g, oracle=shape_a[1] <= 256, oracle_eps=2e-3)


@pytest.mark.parametrize("mode,shape", [("mix", [1024, 2048]), ("mix:dyn", [1000, 2000])])
def test_same_matmul_input(mode, shape):  # :669-679
    g0 = np.random.default_rng(4).normal(0, 0.1, shape).astype(np.float16)
    expect = np.matmul(g0.astype(np.float32), g0.T.astype(np.float32)).astype(np.float16)
    run_graph(mode, lambda k: (lambda a: [(k.store(k.matmul(a, a, False, True)), expect, 2e-3)])(k.load(g0)), oracle_eps=2e-3)


@pytest.mark.parametrize("mode", ["mix", "mix:dyn"])
def test_operand_also_in_epilogue(mode):  # :680-694
    rng = np.random.default_rng(5)
    g0, g1 = rng.normal(0, 0.1, [1024, 1024]).astype(np.float16), rng.normal(0, 0.1, [1024, 1536]).astype(np.float16)
    expect = np.matmul(g0.astype(np.float32), g1.astype(np.float32)).astype(np.float16) + g1

    def g(k):
        b = k.load(g1)
        return [(k.store(k.add(k.matmul(k.load(g0), b, False, False), b)), expect, 2e-3)]
    run_graph(mode, g, oracle_eps=2e-3)


@pytest.mark.parametrize("mix", [False, True])
def test_dynamic_matmul_run_three_times(mix):  # :695-719
    rng = np.random.default_rng(6)
    a, b = rng.normal(0, 0.01, [4096, 4096]).astype(np.float16), rng.normal(0, 0.01, [4096, 4096]).astype(np.float16)
    expect = np.matmul(a.astype(np.float32), b.astype(np.float32))
    Tester.set_lazy_tuning(True)
    try:
        t = Tester("mix:dyn")
        x0, x1 = t.load([], "float16"), t.load([], "float16")
        x2 = t.matmul(x0, x1, False, False)
        if mix:
            x2 = t.add(x2, 0.1)
            expect = expect + 0.1
        x3 = t.store(x2)
        for _ in range(3):
            t.input(x0, a)
            t.input(x1, b)
            t.run()
            assert t.check(x3, expect, 2e-3)
    finally:
        Tester.set_lazy_tuning(False)


def test_single_row_long_k():  # :720-735
    rng = np.random.default_rng(17)
    np_a, np_b = rng.normal(0, 0.1, (1, 80000)).astype(np.float16), rng.normal(0, 0.1, (80000, 256)).astype(np.float16)
    run_graph("mix", lambda k: [(k.store(k.matmul(k.load(np_a), k.load(np_b), False, False)),
                                 np_a.astype(np.float32) @ np_b.astype(np.float32), 2e-3 * 30)], oracle_eps=2e-3 * 30)


@pytest.mark.parametrize("waves", ["4", "8"])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_big_tile_on_four_and_on_eight_waves(monkeypatch, waves, dtype, ta, tb):
    # The 256x256 tile exists on four and on eight waves (the default depends on the layout): both builds, every
    # layout, full tiles with a tail tile in m and n, an epilogue with a bias row and a second operand.
    monkeypatch.setenv("DVM_CUBE_WAVES", waves)
    monkeypatch.setenv("DVM_CUBE_TILE", "256")  # this size would get the 128x128 tile by itself
    m, n, k = 1024 + 40, 2048 + 24, 512
    r = np.random.default_rng(11)
    af = (r.standard_normal([k, m] if ta else [m, k]) / 8).astype(np.float32)
    bf = (r.standard_normal([n, k] if tb else [k, n]) / 8).astype(np.float32)
    bias = r.standard_normal([n]).astype(np.float32)
    other = r.standard_normal([m, n]).astype(np.float32)
    t = Tester("mix")
    if dtype == "bfloat16":
        a16, b16 = Tester.convert_to_bf16(af), Tester.convert_to_bf16(bf)
        a_ref, b_ref = Tester.convert_from_bf16(a16).astype(np.float64), Tester.convert_from_bf16(b16).astype(np.float64)
        x, y = t.load(a16.shape, "bfloat16"), t.load(b16.shape, "bfloat16")
        t.input(x, a16)
        t.input(y, b16)
    else:
        a16, b16 = af.astype(np.float16), bf.astype(np.float16)
        a_ref, b_ref = a16.astype(np.float64), b16.astype(np.float64)
        x, y = t.load(a16), t.load(b16)
    c = t.cast(t.matmul(x, y, ta, tb), "float32")
    out = t.store(t.mul(t.add(c, t.load(bias)), t.load(other)))
    t.run()
    assert ("eight-waves" in t.das()) == (waves == "8"), t.das()
    prod = (a_ref.T if ta else a_ref) @ (b_ref.T if tb else b_ref)
    want = (prod + bias) * other
    got = t.output(out).astype(np.float64)
    assert np.allclose(got, want, rtol=1e-2, atol=1e-2), float(np.abs(got - want).max())


@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_epilogue_with_hardware_approximations(monkeypatch, exact, dtype):
    # An epilogue whose stores are all 16-bit and whose operators are all continuous uses the hardware's exp, log,
    # sqrt and reciprocal (one ulp of fp32); DVM_CUBE_EXACT=1 keeps the library routines. Both must sit within
    # the 16-bit tolerance of the float64 closed form, and a multiply by a constant in front of Exp becomes one
    # instruction with it.
    if exact:
        monkeypatch.setenv("DVM_CUBE_EXACT", "1")
    m, n, k = 300, 520, 192
    r = np.random.default_rng(21)
    af, bf = (r.standard_normal([m, k]) / 8).astype(np.float32), (r.standard_normal([k, n]) / 8).astype(np.float32)
    bias = r.standard_normal([n]).astype(np.float32)
    t = Tester("mix")
    if dtype == "bfloat16":
        a16, b16 = Tester.convert_to_bf16(af), Tester.convert_to_bf16(bf)
        a_ref, b_ref = Tester.convert_from_bf16(a16).astype(np.float64), Tester.convert_from_bf16(b16).astype(np.float64)
        x, y = t.load(a16.shape, "bfloat16"), t.load(b16.shape, "bfloat16")
        t.input(x, a16)
        t.input(y, b16)
        rnd = lambda v: Tester.convert_from_bf16(Tester.convert_to_bf16(v.astype(np.float32))).astype(np.float64)
        eps = 1e-2
    else:
        a16, b16 = af.astype(np.float16), bf.astype(np.float16)
        a_ref, b_ref = a16.astype(np.float64), b16.astype(np.float64)
        x, y = t.load(a16), t.load(b16)
        rnd = lambda v: v.astype(np.float16).astype(np.float64)
        eps = 1e-3
    h = t.add(t.cast(t.matmul(x, y, False, False), "float32"), t.load(bias))
    silu = t.store(t.cast(t.div(h, t.add(t.exp(t.mul(h, -1.0)), 1.0)), dtype))
    other = t.store(t.cast(t.div(t.log(t.add(t.sqrt(t.abs(h)), 1.5)), t.add(t.exp(h), 2.0)), dtype))
    t.run()
    das = t.das()
    assert t.num_launches() == 1, das
    assert ("Exp~" in das and "RDiv~" in das and "Log~" in das and "Sqrt~" in das) == (not exact), das
    assert "acc * #0xbf800000" in das, das  # exp(-h) is one instruction
    hh = rnd(a_ref @ b_ref) + bias
    got = t.output(silu)
    got = Tester.convert_from_bf16(got) if dtype == "bfloat16" else got.astype(np.float32)
    assert np.allclose(got, hh / (1.0 + np.exp(-hh)), rtol=eps, atol=eps)
    got = t.output(other)
    got = Tester.convert_from_bf16(got) if dtype == "bfloat16" else got.astype(np.float32)
    assert np.allclose(got, np.log(np.sqrt(np.abs(hh)) + 1.5) / (np.exp(hh) + 2.0), rtol=eps, atol=eps)


def test_epilogue_with_an_fp32_store_or_a_decision_stays_exact():
    m, n, k = 128, 256, 64
    r = np.random.default_rng(22)
    a16, b16 = (r.standard_normal([m, k]) / 8).astype(np.float16), (r.standard_normal([k, n]) / 8).astype(np.float16)
    prod = a16.astype(np.float64) @ b16.astype(np.float64)
    p16 = prod.astype(np.float16).astype(np.float64)
    # an fp32 store next to the fp16 one
    t = Tester("mix")
    h = t.cast(t.matmul(t.load(a16), t.load(b16), False, False), "float32")
    e = t.exp(h)
    o16, o32 = t.store(t.cast(e, "float16")), t.store(e)
    t.run()
    assert "~" not in t.das(), t.das()
    # the fp16 rounding of the product is the device's (fp32 accumulation): a few elements sit on the other side of a tie
    d32 = np.abs(t.output(o32) - np.exp(p16))
    assert np.mean(d32 > 1e-5 * (1 + np.exp(p16))) < 2e-3 and np.all(d32 < 1e-3)
    assert np.allclose(t.output(o16).astype(np.float64), np.exp(p16), rtol=1e-3, atol=1e-3)
    # a comparison on a value that went through exp
    t = Tester("mix")
    h = t.cast(t.matmul(t.load(a16), t.load(b16), False, False), "float32")
    o = t.store(t.cast(t.select(t.greater(t.exp(h), 1.0), h, t.mul(h, 0.5)), "float16"))
    t.run()
    assert "~" not in t.das(), t.das()
    assert np.allclose(t.output(o).astype(np.float64), np.where(np.exp(p16) > 1.0, p16, p16 * 0.5), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("tile", ["256", "128", "64"])
@pytest.mark.parametrize("m,n", [(256 + 8, 512 + 16), (300, 520), (256, 264), (100, 300), (260, 257), (513, 1024)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_ragged_edge_tiles(monkeypatch, tile, m, n, ta, tb):
    # A ragged tile at the bottom or right edge of an aligned product is moved back inside the output and multiplied
    # like a full tile; its epilogue covers only the part no other tile writes. Shapes with one or both edges ragged,
    # an extent below the tile (guarded path), n not a multiple of 8 (columns cannot move), every tile size; the
    # epilogue reads a second [m, n] operand, so a row or column off by the shift would show.
    monkeypatch.setenv("DVM_CUBE_TILE", tile)
    monkeypatch.setenv("DVM_CUBE_SPLITK", "0")
    k = 192
    r = np.random.default_rng(m * 3 + n)
    a16 = (r.standard_normal([k, m] if ta else [m, k]) / 8).astype(np.float16)
    b16 = (r.standard_normal([n, k] if tb else [k, n]) / 8).astype(np.float16)
    other = r.standard_normal([m, n]).astype(np.float32)
    t = Tester("mix")
    c = t.cast(t.matmul(t.load(a16), t.load(b16), ta, tb), "float32")
    out = t.store(t.add(c, t.load(other)))
    t.run()
    a64, b64 = a16.astype(np.float64), b16.astype(np.float64)
    prod = (a64.T if ta else a64) @ (b64.T if tb else b64)
    got = t.output(out).astype(np.float64)
    bound = 1e-5 + 2.0 ** -11 * np.abs(prod) * 1.01
    assert (np.abs(got - (prod + other)) <= bound).all(), float(np.abs(got - (prod + other)).max())


@pytest.mark.parametrize("mix", [False, True])
def test_dyn_shape_tuning(mix):  # tests/ut/test_matmul.py:697-718: a dynamic kernel run three times with the tuner switched on
    Tester.set_lazy_tuning(True)
    try:
        t = Tester("mix:dyn")
        x0, x1 = t.load([], "float16"), t.load([], "float16")
        x2 = t.matmul(x0, x1, False, False)
        rng = np.random.default_rng(697)
        a = rng.normal(0, 0.01, [4096, 4096]).astype(np.float16)
        b = rng.normal(0, 0.01, [4096, 4096]).astype(np.float16)
        expect = np.matmul(a.astype(np.float32), b.astype(np.float32))
        if mix:
            x2 = t.add(x2, 0.1)
            expect = expect + 0.1
        x3 = t.store(x2)
        for _ in range(3):
            t.input(x0, a)
            t.input(x1, b)
            t.run()
            assert t.check(x3, expect, 2e-3)
    finally:
        Tester.set_lazy_tuning(False)


@pytest.mark.parametrize("ker", ["mix", "split"])
@pytest.mark.parametrize("m,n,k,batch", [(0, 8, 16, ()), (8, 0, 16, ()), (0, 0, 16, ()), (0, 8, 0, ()), (8, 8, 16, (0,))])
def test_matmul_with_an_empty_result(ker, m, n, k, batch):
    a, b = np.ones(batch + (m, k), np.float16), np.ones(batch + (k, n), np.float16)
    t = Tester(ker)
    plain = t.store(t.matmul(t.load(a), t.load(b), False, False))
    fused = t.store(t.add(t.cast(t.matmul(t.load(a), t.load(b), False, False), "float32"), 1.0))
    t.run()
    assert t.output(plain).shape == batch + (m, n) and t.output(fused).shape == batch + (m, n)
    assert plain.shape() == batch + (m, n)


def test_matmul_over_an_empty_k_axis_is_refused_by_name():
    t = Tester("mix")
    t.store(t.matmul(t.load(np.ones([8, 0], np.float16)), t.load(np.ones([0, 8], np.float16)), False, False))
    with pytest.raises(RuntimeError, match="empty k axis"):
        t.codegen()
