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
    assert "rounds per trip" in das_on and "rounds per trip" not in das_off, das_on
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


_PRE_SREG_SCRIPT = r"""
import hashlib, sys
import numpy as np
from dvm_amd.tester import Tester
rng = np.random.default_rng(21)
rows, cols = 5000, 4096  # (one wave per row, four rounds: the statistic lives in an S register)
x = Tester.convert_to_bf16(rng.standard_normal([rows, cols]).astype(np.float32))
w = rng.uniform(0.5, 1.5, [cols]).astype(np.float32)
digest = hashlib.sha256()
fused = 0
for first in ("mul", "add", "sub", "rsub"):
    t = Tester("split")
    lx = t.load(x.shape, "bfloat16"); t.input(lx, x)
    h = t.cast(lx, "float32")
    s = t.div(1.0, t.sqrt(t.add(t.mul(t.sum(t.mul(h, h), (1,), True), 1.0 / cols), 1e-6)))
    y = {"mul": lambda: t.mul(h, s), "add": lambda: t.add(h, s), "sub": lambda: t.sub(h, s), "rsub": lambda: t.sub(s, h)}[first]()
    out = t.store(t.cast(t.mul(y, t.load(w)), "bfloat16"))
    t.run()
    fused += t.das().count("  ; then Mul.fp32 acc, m")
    got = t.output(out)
    digest.update(got.tobytes())
    h64 = Tester.convert_from_bf16(x).astype(np.float64)
    s64 = 1.0 / np.sqrt((h64 * h64).mean(1, keepdims=True) + 1e-6)
    y64 = {"mul": h64 * s64, "add": h64 + s64, "sub": h64 - s64, "rsub": s64 - h64}[first] * w
    assert np.allclose(Tester.convert_from_bf16(got), y64, rtol=1e-2, atol=1e-2), first
print(fused, digest.hexdigest())
"""


def test_an_s_register_binary_in_front_of_a_memory_binary_is_one_instruction():
    # x * rstd * w: the multiply by the S register rides in the dispatch of the multiply by the weight row (VI_PRE_SREG).
    # The same bits as with the instruction stream left as emitted (DVM_VEC_FUSE=0, read once per process: two processes).
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = {}
    for fuse in ("1", "0"):
        env = dict(os.environ, DVM_VEC_FUSE=fuse, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
        p = subprocess.run([sys.executable, "-c", _PRE_SREG_SCRIPT], env=env, cwd=root, capture_output=True, text=True, timeout=100)
        assert p.returncode == 0, p.stderr[-2000:]
        n, digest = p.stdout.split()
        res[fuse] = (int(n), digest)
    assert res["1"][0] >= 3 and res["0"][0] == 0, res  # (one of the four forms may come out with its operands the other way round)
    assert res["1"][1] == res["0"][1]
