"""GPU parity: reduces with few outputs and a long reduced extent, which the host shares between workgroups (a launch
that reduces each part of the reduced index space, a second that reduces over the parts; no atomics, so two runs give
the same bits). Column sums, sums of whole tensors, rows of a million elements, int32 and 16-bit max / min, two
reduces of one input, a reduce beside a pointwise output, forced part counts that do not divide the extent, dynamic
shapes that are shared on one run and not on the next. Expectations: NumPy in float64 (the reference's reduce tests
compare with np.sum at 1e-4, tests/ut/test_reduce.py:25-115), exact for max / min."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def _sum_close(got, x64, axes, scale=1.0):
    want = x64.sum(axis=axes, keepdims=True) * scale
    bound = 1e-5 * np.abs(x64).sum(axis=axes, keepdims=True) * abs(scale) + 1e-6  # fp32 partial sums, fp64 inside a part
    return (np.abs(got.astype(np.float64).reshape(want.shape) - want) <= bound).all()


@pytest.mark.parametrize("shape,axes", [((4096, 4096), (0,)), ((4096, 4100), (0,)), ((1 << 20, 7), (0,)), ((100000, 128), (0,)),
                                        ((7, 1 << 20), (1,)), ((1 << 24,), (0,)), ((3, 1000003), (1,)), ((64, 512, 1024), (1,)),
                                        ((2, 3, 40000, 5), (2,)), ((2000, 3, 1000), (0, 2)), ((513, 70001), (0, 1))])
@pytest.mark.parametrize("keepdims", [True, False])
def test_sum_with_few_outputs(shape, axes, keepdims):
    rng = np.random.default_rng(len(shape) * 100 + axes[0])
    x = rng.standard_normal(shape, dtype=np.float32)
    t = Tester("split")
    out = t.store(t.mul(t.sum(t.load(x), axes, keepdims), 0.5))
    t.run()
    das = t.das()
    assert "shared-reduce parts=" in das and t.num_launches() == 2, das
    got = t.output(out)
    assert got.shape == x.sum(axis=axes, keepdims=keepdims).shape
    assert _sum_close(got, x.astype(np.float64), axes, 0.5)


@pytest.mark.parametrize("dtype", ["int32", "float16", "float32"])
@pytest.mark.parametrize("shape,axes", [((1 << 20, 7), (0,)), ((5, 300000), (1,)), ((1 << 22,), (0,))])
def test_max_and_min_are_exact(dtype, shape, axes):
    rng = np.random.default_rng(7)
    if dtype == "int32":
        x = rng.integers(-(1 << 31), (1 << 31) - 1, shape, dtype=np.int64).astype(np.int32)
    else:
        x = (rng.standard_normal(shape) * 100).astype(dtype)
    t = Tester("split")
    lx = t.load(x)
    hi, lo = t.store(t.max(lx, axes, True)), t.store(t.min(lx, axes, True))
    t.run()
    assert t.das().count("shared-reduce parts=") >= 1, t.das()
    assert np.array_equal(t.output(hi), x.max(axis=axes, keepdims=True))
    assert np.array_equal(t.output(lo), x.min(axis=axes, keepdims=True))


def test_two_reduces_of_one_input_and_what_follows_them():
    # mean and variance of each column of a [200000, 96] tensor: both reduces are shared alike, the arithmetic on their
    # results rides in the launch that reduces over the parts
    rng = np.random.default_rng(11)
    x = (rng.standard_normal([200000, 96]) * 3 + 1).astype(np.float32)
    n = x.shape[0]
    t = Tester("split")
    lx = t.load(x)
    mean = t.mul(t.sum(lx, (0,), True), 1.0 / n)
    ex2 = t.mul(t.sum(t.mul(lx, lx), (0,), True), 1.0 / n)
    var = t.store(t.sub(ex2, t.mul(mean, mean)))
    m = t.store(mean)
    t.run()
    das = t.das()
    assert das.count("shared-reduce parts=") == 1 and t.num_launches() == 2, das
    x64 = x.astype(np.float64)
    assert np.allclose(t.output(m), x64.mean(0, keepdims=True), rtol=1e-5, atol=1e-5)
    assert np.allclose(t.output(var), x64.var(0, keepdims=True), rtol=1e-4, atol=1e-4)


def test_a_reduce_whose_consumer_walks_the_input_again():
    # softmax over rows of 262144 elements, three rows: max and sum are both shared (three workgroups would walk a
    # megabyte each three times: 180 us in one launch, 110 us in five); exp(x - max) reads the maxima from memory in the
    # launch that sums its parts, and is stored there for the launch that divides
    rng = np.random.default_rng(12)
    x = rng.standard_normal([3, 1 << 18]).astype(np.float32)
    t = Tester("split")
    lx = t.load(x)
    e = t.exp(t.sub(lx, t.max(lx, (1,), True)))
    out = t.store(t.div(e, t.sum(e, (1,), True)))
    t.run()
    das = t.das()
    assert das.count("shared-reduce parts=") == 2 and t.num_launches() == 5, das
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(1, keepdims=True))
    assert np.allclose(t.output(out), e64 / e64.sum(1, keepdims=True), rtol=1e-4, atol=1e-9)


@pytest.mark.parametrize("shape", [(4096, 1024), (32000, 512)])
def test_softmax_over_the_outer_axis(shape):
    # max and sum over axis 0 with consumers on the whole tensor: two shared reduces, their results read from memory
    rng = np.random.default_rng(17)
    x = rng.standard_normal(shape).astype(np.float32)
    t = Tester("split")
    lx = t.load(x)
    e = t.exp(t.sub(lx, t.max(lx, (0,), True)))
    out = t.store(t.div(e, t.sum(e, (0,), True)))
    t.run()
    assert t.das().count("shared-reduce parts=") == 2, t.das()
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(0, keepdims=True))
    assert np.allclose(t.output(out), e64 / e64.sum(0, keepdims=True), rtol=1e-4, atol=1e-9)


def test_a_pointwise_output_beside_a_shared_reduce():
    rng = np.random.default_rng(13)
    x = rng.standard_normal([300000, 40]).astype(np.float32)
    t = Tester("split")
    y = t.add(t.load(x), 1.0)
    full = t.store(y)
    col = t.store(t.sum(y, (0,), False))
    t.run()
    # (the pointwise output is stored by the launch that reduces the parts: every element of y lies in exactly one part)
    assert "shared-reduce parts=" in t.das() and t.num_launches() == 2, t.das()
    assert np.array_equal(t.output(full), x + np.float32(1.0))
    assert _sum_close(t.output(col), (x + np.float32(1.0)).astype(np.float64), (0,))


@pytest.mark.parametrize("parts", ["3", "7", "64"])
@pytest.mark.parametrize("shape,axes", [((1000, 24), (0,)), ((5, 4099), (1,)), ((77777,), (0,))])
def test_forced_part_counts_that_do_not_divide_the_extent(monkeypatch, parts, shape, axes):
    # the last part is short, and with 64 parts of a short extent some are empty: they contribute the reduce's identity
    monkeypatch.setenv("DVM_RED_SPLIT", parts)
    rng = np.random.default_rng(int(parts) + shape[0])
    x = rng.standard_normal(shape).astype(np.float32)
    t = Tester("split")
    lx = t.load(x)
    s, hi = t.store(t.sum(lx, axes, True)), t.store(t.max(lx, axes, True))
    t.run()
    assert "shared-reduce parts=" in t.das(), t.das()
    assert _sum_close(t.output(s), x.astype(np.float64), axes)
    assert np.array_equal(t.output(hi), x.max(axis=axes, keepdims=True))


def test_same_bits_on_every_run_and_against_the_single_launch(monkeypatch):
    rng = np.random.default_rng(14)
    x = rng.standard_normal([1 << 21, 3]).astype(np.float32)
    outs = []
    for split in [None, None, "0"]:
        if split is not None:
            monkeypatch.setenv("DVM_RED_SPLIT", split)
        t = Tester("split")
        out = t.store(t.sum(t.load(x), (0,), True))
        t.run()
        assert ("shared-reduce" in t.das()) == (split is None)
        outs.append(t.output(out).copy())
    assert np.array_equal(outs[0], outs[1])
    assert np.allclose(outs[0], outs[2], rtol=1e-5, atol=1e-3)  # partial sums rounded to fp32 once more


def test_dynamic_shapes_shared_on_one_run_and_not_on_the_next():
    rng = np.random.default_rng(15)
    t = Tester("split:dyn")
    lx = t.load([-1, -1], "float32")
    out = t.store(t.sum(lx, (0,), True))
    for rows, cols, shared in [(400000, 16, True), (64, 16, False), (300, 300000, False), (250000, 130, True), (400000, 16, True)]:
        x = rng.standard_normal([rows, cols]).astype(np.float32)
        t.input(lx, x)
        t.run()
        assert ("shared-reduce" in t.das()) == shared, (rows, cols, t.das())
        assert _sum_close(t.output(out), x.astype(np.float64), (0,)), (rows, cols)


def test_consumers_larger_than_the_reduce_get_launches_of_their_own():
    # (x - mean) / sqrt(var + eps) over axis 0 of [8192, 1024] (a batch-norm in channels-last layout): both sums are
    # shared between workgroups; the launches that reduce over the parts hold the per-column arithmetic only, x - mean
    # and the division read their results from memory (in one launch with them, every element of x would reduce the
    # 128 partial sums of its column again)
    rng = np.random.default_rng(16)
    x = (rng.standard_normal([8192, 1024]) * 2 + 0.5).astype(np.float32)
    t = Tester("split")
    lx = t.load(x)
    mean = t.mul(t.sum(lx, (0,), True), 1.0 / 8192)
    d = t.sub(lx, mean)
    var = t.mul(t.sum(t.mul(d, d), (0,), True), 1.0 / 8192)
    out = t.store(t.div(d, t.sqrt(t.add(var, 1e-5))))
    t.run()
    das = t.das()
    assert das.count("shared-reduce parts=") == 2 and t.num_launches() == 5, das
    for entry in das.split("== sub-kernel")[1:]:
        head = entry.splitlines()[1]
        if "sched=reduce-y" in head and "shared-reduce" not in head:  # a launch that reduces over the parts
            assert "kept=128 " in head, head
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(0, keepdims=True)) / np.sqrt(x64.var(0, keepdims=True) + 1e-5)
    assert np.allclose(t.output(out), want, rtol=1e-5, atol=1e-5), float(np.abs(t.output(out) - want).max())


def _channels_last_batch_norm(t, x, g, b):
    n = x.shape[0] * x.shape[1] * x.shape[2]
    lx, lg, lb = t.load(x), t.load(g), t.load(b)
    mean = t.mul(t.sum(lx, (0, 1, 2), True), 1.0 / n)
    var = t.sub(t.mul(t.sum(t.mul(lx, lx), (0, 1, 2), True), 1.0 / n), t.mul(mean, mean))
    scale = t.div(lg, t.sqrt(t.add(var, 1e-5)))
    return t.store(t.add(t.mul(lx, scale), t.sub(lb, t.mul(mean, scale)))), t.store(mean)


@pytest.mark.parametrize("shape", [(32, 56, 56, 256), (8, 28, 28, 96), (4, 57, 31, 40)])
def test_batch_norm_channels_last(monkeypatch, shape):
    # [N, H, W, C] with the statistics over N, H, W: the innermost axis is kept, the reduce is shared between workgroups.
    # Its partial results are stored with the parts innermost, so the launch over the parts reduces along rows (the sweep
    # build where the part count allows); with DVM_RED_SPLIT_TURN=0 it walks them outermost. Both against float64.
    rng = np.random.default_rng(shape[3])
    x = (rng.standard_normal(shape, dtype=np.float32) * 2.0 + 3.0).astype(np.float32)
    g = rng.uniform(0.5, 1.5, [1, 1, 1, shape[3]]).astype(np.float32)
    b = rng.normal(0, 0.1, [1, 1, 1, shape[3]]).astype(np.float32)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean((0, 1, 2), keepdims=True)) / np.sqrt(x64.var((0, 1, 2), keepdims=True) + 1e-5) * g + b
    for turn in ("1", "0"):
        monkeypatch.setenv("DVM_RED_SPLIT_TURN", turn)
        monkeypatch.setenv("DVM_RED_SPLIT", "64" if shape[0] < 32 else "-1")
        t = Tester("split")
        y, mean = _channels_last_batch_norm(t, x, g, b)
        t.run()
        das = t.das()
        assert "shared-reduce parts=" in das and t.num_launches() == 3, das
        if turn == "1":
            assert "sched=reduce-x" in das and "gather" in das, das  # rows of partial results, written scattered
        else:
            assert "sched=reduce-x" not in das, das
        assert np.allclose(t.output(mean), x64.mean((0, 1, 2), keepdims=True), rtol=1e-5, atol=1e-5)
        assert np.allclose(t.output(y), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,cols,parts", [(4096, 512, 16), (4100, 520, 16), (1031, 64, 4), (30000, 8, 32), (257, 4096, 2)])
@pytest.mark.parametrize("kind", ["sum", "sumsq", "max"])
def test_column_reduces_fetch_several_rounds_per_trip(monkeypatch, rows, cols, parts, kind):
    # a sweep that is one load and one reduce takes four rounds per trip to memory on the schedule that keeps the
    # innermost axis: row counts that leave one, two and three rounds for the last trip, ragged columns, rows past the end
    monkeypatch.setenv("DVM_RED_SPLIT", str(parts))
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal([rows, cols], dtype=np.float32)
    t = Tester("split")
    lx = t.load(x)
    if kind == "sum":
        o = t.store(t.sum(lx, (0,), True))
    elif kind == "sumsq":
        o = t.store(t.sum(t.mul(lx, lx), (0,), True))
    else:
        o = t.store(t.max(lx, (0,), True))
    t.run()
    das = t.das()
    assert "fetches several rounds per trip" in das, das
    got = t.output(o)
    x64 = x.astype(np.float64)
    if kind == "max":
        assert np.array_equal(got, x.max(0, keepdims=True))
    elif kind == "sum":
        assert _sum_close(got, x64, (0,))
    else:
        assert _sum_close(got, x64 * x64, (0,))
    # no atomics anywhere: a second run gives the same bits
    t2 = Tester("split")
    l2 = t2.load(x)
    o2 = t2.store(t2.sum(l2, (0,), True) if kind == "sum" else (t2.sum(t2.mul(l2, l2), (0,), True) if kind == "sumsq" else t2.max(l2, (0,), True)))
    t2.run()
    assert np.array_equal(got, t2.output(o2))
