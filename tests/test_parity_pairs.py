"""GPU parity of the loads that take work along: a load that fetches the next instruction's operand in the same
trip (VI_LD_PAIR), the load of a statistics sweep that fetches two rounds per trip and does the reduce (VI_LD_RED2),
and rounds parked behind the instruction two sweeps share (VI_LD_KEEP_* with a prefix). Each is an optimisation of
the interpreter only: with DVM_VEC_PAIR=0 the same programs run instruction by instruction, and both must give
the same bits (the reduce accumulates in the order of the rounds either way) and agree with the float64 closed
forms. Shapes are chosen so that sweeps have one, two, odd and even numbers of rounds and ragged last rounds."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def _run(monkeypatch, pair, build):
    if pair:
        monkeypatch.delenv("DVM_VEC_PAIR", raising=False)
    else:
        monkeypatch.setenv("DVM_VEC_PAIR", "0")
    t = Tester("split")
    outs = build(t)
    t.run()
    return [t.output(o) for o in outs], t.das()


@pytest.mark.parametrize("shape", [[3, 40], [5, 1000], [7, 5000], [2, 16384], [9, 33000], [300, 4096], [1, 200001]])
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_statistics_sweeps_two_rounds_per_trip(monkeypatch, shape, dtype):
    rng = np.random.default_rng(shape[1])
    x = rng.standard_normal(shape, dtype=np.float32).astype(dtype)

    def build(t):
        lx = t.load(x)
        xf = t.cast(lx, "float32") if dtype != "float32" else lx
        mean = t.mul(t.sum(xf, (1,), True), 1.0 / shape[1])
        var = t.sub(t.mul(t.sum(t.mul(xf, xf), (1,), True), 1.0 / shape[1]), t.mul(mean, mean))
        return [t.store(t.div(t.sub(xf, mean), t.sqrt(t.add(var, 1e-5)))), t.store(mean)]

    (a, am), das_on = _run(monkeypatch, True, build)
    (b, bm), das_off = _run(monkeypatch, False, build)
    assert "two rounds per trip" in das_on and "two rounds per trip" not in das_off, das_on
    assert np.array_equal(a, b) and np.array_equal(am, bm)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    assert np.allclose(a, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("rows,cols", [(1, 4096), (5, 4096), (64, 4096), (700, 4096), (4100, 4096), (33, 1000), (4, 24000)])
def test_residual_norm_pairs_loads_and_parks_the_sum(monkeypatch, rows, cols):
    rng = np.random.default_rng(rows * 7 + cols)
    xs = Tester.convert_to_bf16(rng.standard_normal([rows, cols], dtype=np.float32))
    rs = Tester.convert_to_bf16(rng.standard_normal([rows, cols], dtype=np.float32))
    wv = rng.uniform(0.9, 1.1, [cols]).astype(np.float32)

    def build(t):
        x, r = t.load(xs.shape, "bfloat16"), t.load(rs.shape, "bfloat16")
        t.input(x, xs)
        t.input(r, rs)
        hf = t.cast(t.add(x, r), "float32")
        rstd = t.div(1.0, t.sqrt(t.add(t.mul(t.sum(t.mul(hf, hf), (1,), True), 1.0 / cols), 1e-6)))
        return [t.store(t.cast(t.mul(t.mul(hf, rstd), t.load(wv)), "bfloat16"))]

    (a,), das_on = _run(monkeypatch, True, build)
    (b,), das_off = _run(monkeypatch, False, build)
    assert "in the same trip" in das_on and "in the same trip" not in das_off, das_on
    assert np.array_equal(a, b)
    hh = Tester.convert_from_bf16(Tester.convert_to_bf16(Tester.convert_from_bf16(xs) + Tester.convert_from_bf16(rs))).astype(np.float64)
    want = hh / np.sqrt((hh * hh).mean(1, keepdims=True) + 1e-6) * wv
    assert np.allclose(Tester.convert_from_bf16(a), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("shape", [[1000], [33, 77], [4, 3, 50, 50]])
def test_pointwise_pairs(monkeypatch, shape):
    rng = np.random.default_rng(len(shape))
    x, y, z = (rng.standard_normal(shape, dtype=np.float32) for _ in range(3))

    def build(t):
        return [t.store(t.add(t.mul(t.load(x), t.load(y)), t.load(z)))]

    (a,), das_on = _run(monkeypatch, True, build)
    (b,), _ = _run(monkeypatch, False, build)
    assert "in the same trip" in das_on
    assert np.array_equal(a, b) and np.array_equal(a, x * y + z)


def test_parked_sum_survives_a_mixed_type_pair(monkeypatch):
    # fp16 + fp32 operands: the pair is fetched one after the other, the parked value is fp32 (two planes)
    rng = np.random.default_rng(5)
    x = rng.standard_normal([40, 3000], dtype=np.float32).astype(np.float16)
    y = rng.standard_normal([40, 3000], dtype=np.float32)

    def build(t):
        s = t.add(t.cast(t.load(x), "float32"), t.load(y))
        return [t.store(t.div(s, t.sum(t.abs(s), (1,), True)))]

    (a,), _ = _run(monkeypatch, True, build)
    (b,), _ = _run(monkeypatch, False, build)
    assert np.array_equal(a, b)
    s64 = x.astype(np.float64) + y.astype(np.float64)
    assert np.allclose(a, s64 / np.abs(s64).sum(1, keepdims=True), rtol=1e-4, atol=1e-6)
