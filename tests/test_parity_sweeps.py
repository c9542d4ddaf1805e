"""GPU parity of the sweep build of the vector VM (dvm_vm_vec_rx_sw): programs that reduce the innermost axis and
whose sweeps are chains of float arithmetic behind one load run their rounds in native loops there. The generic
kernel runs the same instruction words (DVM_VEC_SWEEPS=0), and both must give the same bits: the reduce
accumulates per lane in the order of the rounds either way. Each graph is also checked against its float64 closed
form. Shapes cover rows of one wave and of a whole workgroup, several rows per wave, ragged last rounds, rounds
that are empty for some waves, two reduced axes (a channel of an NCHW tensor) and reduces shared between workgroups.

The host's decision (which programs carry the flag) is checked without a GPU in test_host.py."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def _run(monkeypatch, sweeps, build, ker="split"):
    if sweeps:
        monkeypatch.delenv("DVM_VEC_SWEEPS", raising=False)
    else:
        monkeypatch.setenv("DVM_VEC_SWEEPS", "0")
    t = Tester(ker)
    outs = build(t)
    t.run()
    return [t.output(o) for o in outs], t.das()


@pytest.mark.parametrize("shape", [[3, 40], [5, 1000], [7, 5000], [2, 16384], [9, 33000], [300, 4096], [1, 200001], [4100, 2048], [64, 4104]])
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
def test_layer_norm_rows(monkeypatch, shape, dtype):
    rng = np.random.default_rng(shape[0] * 131 + shape[1])
    xf32 = rng.standard_normal(shape, dtype=np.float32)
    x = Tester.convert_to_bf16(xf32) if dtype == "bfloat16" else xf32.astype(dtype)
    w = rng.uniform(0.5, 1.5, [shape[1]]).astype(np.float32)
    b = rng.normal(0, 0.1, [shape[1]]).astype(np.float32)

    def build(t):
        lx = t.load(x.shape, dtype)
        t.input(lx, x)
        xf = t.cast(lx, "float32") if dtype != "float32" else lx
        mean = t.mul(t.sum(xf, (1,), True), 1.0 / shape[1])
        xc = t.sub(xf, mean)
        var = t.mul(t.sum(t.mul(xc, xc), (1,), True), 1.0 / shape[1])
        y = t.add(t.mul(t.div(xc, t.sqrt(t.add(var, 1e-5))), t.load(w)), t.load(b))
        return [t.store(y), t.store(mean), t.store(var)]

    # (a row that fits one round keeps its values in the accumulator between the sweeps: not the sweep build's case,
    # so the flag is only asserted for the rows that take several rounds whatever the team)
    (y, mean, var), das_on = _run(monkeypatch, True, build)
    off, _ = _run(monkeypatch, False, build)
    for p, q in zip((y, mean, var), off):
        assert np.array_equal(p, q), das_on
    if shape[1] > 2048 * 8:
        assert "reduce-x sweeps" in das_on, das_on
    x64 = (Tester.convert_from_bf16(x) if dtype == "bfloat16" else x).astype(np.float64)
    assert np.allclose(mean, x64.mean(1, keepdims=True), rtol=1e-5, atol=1e-5)
    want = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5) * w + b
    assert np.allclose(y, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("rows,cols", [(1, 4096), (5, 4096), (64, 4096), (700, 4096), (2500, 4096), (4100, 4096), (8192, 4096), (33, 1000), (4, 24000), (3000, 8192)])
def test_residual_rmsnorm(monkeypatch, rows, cols):
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

    a, das_on = _run(monkeypatch, True, build)
    b, _ = _run(monkeypatch, False, build)
    assert np.array_equal(a[0], b[0]), das_on
    if rows >= 2048 or cols > 8192:  # rows of one or two waves, or of several rounds: the sweep build's case
        assert "reduce-x sweeps" in das_on, das_on
    hh = Tester.convert_from_bf16(Tester.convert_to_bf16(Tester.convert_from_bf16(xs) + Tester.convert_from_bf16(rs))).astype(np.float64)
    want = hh / np.sqrt((hh * hh).mean(1, keepdims=True) + 1e-6) * wv
    assert np.allclose(Tester.convert_from_bf16(a[0]), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("shape", [[2, 3, 5, 7], [4, 16, 14, 14], [32, 8, 56, 56], [3, 5, 33, 31], [1, 2, 300, 300]])
@pytest.mark.parametrize("two_pass", [False, True])
def test_batch_norm_channels(monkeypatch, shape, two_pass):
    n, c, h, w = shape
    rng = np.random.default_rng(n * 1000 + c * 100 + h)
    x = (rng.standard_normal(shape, dtype=np.float32) * 2.0 + 3.0).astype(np.float32)
    g = rng.uniform(0.5, 1.5, [1, c, 1, 1]).astype(np.float32)
    b = rng.normal(0, 0.1, [1, c, 1, 1]).astype(np.float32)
    inv = 1.0 / (n * h * w)

    def build(t):
        lx, lg, lb = t.load(x), t.load(g), t.load(b)
        mean = t.mul(t.sum(lx, (0, 2, 3), True), inv)
        if two_pass:  # the reference's example: the variance from the centred values
            xc = t.sub(lx, mean)
            var = t.mul(t.sum(t.mul(xc, xc), (0, 2, 3), True), inv)
            y = t.add(t.mul(t.div(xc, t.sqrt(t.add(var, 1e-5))), lg), lb)
        else:
            var = t.sub(t.mul(t.sum(t.mul(lx, lx), (0, 2, 3), True), inv), t.mul(mean, mean))
            scale = t.div(lg, t.sqrt(t.add(var, 1e-5)))
            y = t.add(t.mul(lx, scale), t.sub(lb, t.mul(mean, scale)))
        return [t.store(y), t.store(mean)]

    a, das_on = _run(monkeypatch, True, build)
    bb, _ = _run(monkeypatch, False, build)
    for p, q in zip(a, bb):
        assert np.array_equal(p, q), das_on
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean((0, 2, 3), keepdims=True)) / np.sqrt(x64.var((0, 2, 3), keepdims=True) + 1e-5) * g + b
    assert np.allclose(a[0], want, rtol=1e-4 if not two_pass else 2e-5, atol=1e-4 if not two_pass else 2e-5)


@pytest.mark.parametrize("shape", [[16, 3000], [300, 5000], [2, 70000], [2100, 2048]])
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_softmax_rows(monkeypatch, shape, dtype):
    rng = np.random.default_rng(shape[0] + shape[1])
    x = (rng.standard_normal(shape, dtype=np.float32) * 3.0).astype(dtype)

    def build(t):
        lx = t.load(x)
        xf = t.cast(lx, "float32") if dtype != "float32" else lx
        e = t.exp(t.sub(xf, t.max(xf, (1,), True)))
        y = t.div(e, t.sum(e, (1,), True))
        return [t.store(t.cast(y, dtype) if dtype != "float32" else y)]

    a, das_on = _run(monkeypatch, True, build)
    b, _ = _run(monkeypatch, False, build)
    assert np.array_equal(a[0], b[0]), das_on
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(1, keepdims=True))
    tol = 2e-3 if dtype == "float16" else 1e-5
    assert np.allclose(a[0], e / e.sum(1, keepdims=True), rtol=tol, atol=tol)


def test_shared_reduce_runs_its_parts_on_the_sweep_build(monkeypatch):
    # few rows, long: the reduce is shared between workgroups (parts), the launch over the parts reduces the innermost axis
    rng = np.random.default_rng(11)
    x = rng.standard_normal([4, 1 << 20], dtype=np.float32)

    def build(t):
        lx = t.load(x)
        return [t.store(t.sum(lx, (1,), True)), t.store(t.max(lx, (1,), True))]

    a, das_on = _run(monkeypatch, True, build)
    b, _ = _run(monkeypatch, False, build)
    for p, q in zip(a, b):
        assert np.array_equal(p, q), das_on
    assert "reduce-x sweeps" in das_on and "parts=" in das_on, das_on
    assert np.allclose(a[0], x.astype(np.float64).sum(1, keepdims=True), rtol=1e-5, atol=1e-3)
    assert np.array_equal(a[1], x.max(1, keepdims=True))


def test_unaligned_rows_and_addresses_fall_back_to_the_generic_kernel(monkeypatch):
    # rows of 4097 elements: no row but the first starts on 16 bytes, so the program never carries the flag
    rng = np.random.default_rng(5)
    x = rng.standard_normal([2200, 4097], dtype=np.float32)

    def build(t):
        lx = t.load(x)
        m = t.mul(t.sum(lx, (1,), True), 1.0 / 4097)
        return [t.store(t.sub(lx, m))]

    a, das_on = _run(monkeypatch, True, build)
    assert "reduce-x sweeps" not in das_on, das_on
    assert np.allclose(a[0], x - x.astype(np.float64).mean(1, keepdims=True), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("sweeps", [True, False])
@pytest.mark.parametrize("first", ["times a number", "plus a number", "plus a tensor"])
@pytest.mark.parametrize("n", [40000, 70001])
def test_parked_rounds_hold_the_value_behind_the_first_instruction(monkeypatch, sweeps, first, n):
    # Both sweeps open with [load x] [one float binary]: the rounds that stay in local memory hold that binary's
    # result, whatever its operand is. (With a number as the operand the generic kernel once parked the value behind
    # the instruction after it.) A store of a V register between the sweeps keeps the program off the sweep build.
    rng = np.random.default_rng(n)
    x, y = rng.uniform(0.25, 2.0, [n]).astype(np.float32), rng.uniform(0.25, 2.0, [n]).astype(np.float32)
    head = {"times a number": lambda k, a, b: k.mul(a, -1.0), "plus a number": lambda k, a, b: k.add(a, 0.75),
            "plus a tensor": lambda k, a, b: k.add(a, b)}[first]
    h64 = {"times a number": -x.astype(np.float64), "plus a number": x.astype(np.float64) + 0.75,
           "plus a tensor": x.astype(np.float64) + y}[first]
    v64 = h64 * x
    want = v64.max() - v64 / (np.abs(v64) + 0.5)

    def build(k):
        a, b = k.load(x), k.load(y)
        v = k.mul(head(k, a, b), a)
        top = k.max(v, (0,), True)
        return [k.store(k.sub(top, k.div(v, k.add(k.abs(v), 0.5))))]
    (out,), das = _run(monkeypatch, sweeps, build)
    assert "parks its first" in das, das
    assert np.allclose(out, want, rtol=1e-5, atol=1e-6), (np.abs(out - want).max(), das)


@pytest.mark.parametrize("sweeps", [True, False])
@pytest.mark.parametrize("rows,cols", [(500, 4096), (37, 1000), (3, 20000)])
def test_operand_read_inside_a_per_output_run_and_again_behind_it(monkeypatch, sweeps, rows, cols):
    # A per-row value is loaded inside a run that only the first wave of the workgroup executes, stored, and loaded
    # again behind the run: the waves that skipped the run have to compute that operand's offsets themselves.
    # (They once reused offsets they never had, and every row but the first read the first row's value.)
    rng = np.random.default_rng(rows)
    c = rng.uniform(0.25, 2.0, [rows, 1]).astype(np.float32)
    x = rng.uniform(0.25, 2.0, [rows, cols]).astype(np.float16)
    e = np.exp(c.astype(np.float64) * 0.125)
    d = x.astype(np.float64) - e * c

    def build(k):
        cv = k.load(c)
        ev = k.exp(k.mul(cv, 0.125))
        diff = k.sub(k.cast(k.load(x), "float32"), k.mul(ev, cv))
        return [k.store(k.cast(k.cast(ev, "float16"), "float32")), k.store(diff), k.store(k.sum(diff, (1,), True))]
    (o0, o1, o2), das = _run(monkeypatch, sweeps, build)
    assert "per-output run" in das, das
    assert np.allclose(o0, e.astype(np.float16).astype(np.float32), rtol=1e-3)
    assert np.allclose(o1, d, rtol=1e-5, atol=1e-5), np.abs(o1 - d).max()
    assert np.allclose(o2, d.sum(1, keepdims=True), rtol=1e-4, atol=1e-3)
