"""GPU parity: GroupedMatMul, restating tests/ut/test_gmm.py of the reference (cited per test): the groups split the rows
of the left operand (group_type 0: one weight matrix per group, result [m, n]) or the k axis (group_type 2: result
[groups, m, n]); the list of bounds (or sizes) is an int64 tensor read on the device. Expectations are the reference's
own NumPy rules (np_gmm_split_m / np_gmm_split_k, :25-76); the shapes the scalar CPU oracle finishes in seconds also run
on it. Tolerances as there: 1e-3 for fp16 outputs, 3e-3 for bf16."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def rng(seed=0):
    return np.random.default_rng(seed)


def gmm_split_m(x, w, b, bounds):  # tests/ut/test_gmm.py:25-51
    outs, lo = [], 0
    for i, g in enumerate(bounds):
        out_i = x[lo:g].astype(np.float32) @ w[i].astype(np.float32)
        if b is not None:
            out_i += b[i]
        outs.append(out_i)
        lo = g
    return np.concatenate(outs, axis=0)


def gmm_split_k(x, w, b, bounds):  # :54-76
    out = np.zeros((len(bounds), x.shape[0], w.shape[1]))
    lo = 0
    for i, g in enumerate(bounds):
        out[i] = x[:, lo:g].astype(np.float32) @ w[lo:g, :].astype(np.float32)
        if b is not None:
            out[i] += b[i]
        lo = g
    return out


def rows_of(k, out, upto):
    """The rows a split over m writes: everything below the last bound."""
    return out[:upto]


@pytest.mark.parametrize("m, n, k, bounds, oracle", [
    (2333, 1111, 2222, [777, 2333], False), (4096, 4096, 4096, [10, 256, 256, 3000, 4096], False),
    (4352, 2048, 4096, [0, 10, 256, 256, 777, 1024, 2051, 3000, 4096, 4352], False), (300, 96, 128, [7, 7, 130, 300], True)])
@pytest.mark.parametrize("trans", [[False, True], [True, True], [False, False], [True, False]])
def test_gmm(m, n, k, bounds, trans, oracle):  # :79-106 (the third shape with an eighth of its k axis)
    g = len(bounds)
    x = Tester.fast_random_normal(0, 0.01, [k, m] if trans[0] else [m, k]).astype(np.float16)
    w = Tester.fast_random_normal(0, 0.01, [g, n, k] if trans[1] else [g, k, n]).astype(np.float16)
    gl = np.array(bounds, np.int64)
    expect = gmm_split_m(x.T if trans[0] else x, w.transpose(0, 2, 1) if trans[1] else w, None, gl)
    run_graph("mix", lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x), kk.load(w), trans[0], trans[1], None, kk.load(gl), 0)), expect, 1e-3)],
              oracle=oracle)


@pytest.mark.parametrize("mode", ["mix", "eager"])
@pytest.mark.parametrize("m, n, k, bounds", [(1024, 4096, 512, [512, 1024]), (4096, 4096, 4096, [10, 500, 1024, 2048, 3333, 4096])])
def test_gmm_bias(mode, m, n, k, bounds):  # :109-134
    g = len(bounds)
    x = Tester.fast_random_normal(0, 0.01, [m, k]).astype(np.float16)
    w = Tester.fast_random_normal(0, 0.01, [g, k, n]).astype(np.float16)
    bias = Tester.fast_random_normal(0, 0.01, [g, n]).astype(np.float16)
    gl = np.array(bounds, np.int64)
    expect = gmm_split_m(x, w, bias, gl)
    run_graph(mode, lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x), kk.load(w), False, False, kk.load(bias), kk.load(gl), 0)), expect, 1e-3)],
              oracle=False)


def test_gmm_bias_bf16():  # :137-158
    m, n, k, bounds = 1024, 4096, 512, [512, 1024]
    x = Tester.fast_random_normal(0, 0.01, [m, k]).astype(np.float32)
    w = Tester.fast_random_normal(0, 0.01, [2, k, n]).astype(np.float32)
    bias = Tester.fast_random_normal(0, 0.01, [2, n]).astype(np.float32)
    gl = np.array(bounds, np.int64)
    expect = gmm_split_m(x, w, bias, gl)
    run_graph("mix", lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x, "bfloat16"), kk.load(w, "bfloat16"), False, False,
                                                             kk.load(bias, "bfloat16"), kk.load(gl), 0)), expect, 3e-3)], oracle=False)


@pytest.mark.parametrize("groups", [255, 256, 1024])
def test_gmm_group_count_bf16(groups):  # :161-177
    m, n, k = 2048, 64, 64
    gl = np.arange(1, groups + 1, dtype=np.int64) * m // groups
    x = Tester.fast_random_normal(0, 0.01, [m, k]).astype(np.float32)
    w = Tester.fast_random_normal(0, 0.01, [groups, k, n]).astype(np.float32)
    expect = gmm_split_m(x, w, None, gl)
    run_graph("mix", lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x, "bfloat16"), kk.load(w, "bfloat16"), False, False, None, kk.load(gl), 0)),
                                  expect, 3e-3)])


def test_gmm_sizes_int32_list_bias_and_an_epilogue_on_the_oracle():
    # the list as sizes (group_list_type 1) and as int32; a bias row per group; an activation behind the product
    m, n, k = 700, 192, 256
    sizes = [0, 130, 1, 255, 0, 314]
    x = rng(1).normal(0, 0.1, [m, k]).astype(np.float16)
    w = rng(2).normal(0, 0.1, [len(sizes), k, n]).astype(np.float16)
    bias = rng(3).normal(0, 0.1, [len(sizes), n]).astype(np.float16)
    bounds = np.cumsum(sizes)
    want = np.maximum(gmm_split_m(x, w, bias, bounds).astype(np.float16).astype(np.float32) * np.float32(0.5), 0)
    for list_dtype in (np.int64, np.int32):
        gl = np.array(sizes, list_dtype)

        def build(kk):
            r = kk.grouped_matmul(kk.load(x), kk.load(w), False, False, kk.load(bias), kk.load(gl), 0, 1)
            return [(kk.store(kk.maximum(kk.mul(kk.cast(r, "float32"), 0.5), 0.0)), want, 1e-3)]

        t = run_graph("mix", build, oracle_eps=1e-3)  # (an fp16 product behind the fp32 store: the order of the fp32 sums shows as one fp16 step)
        assert t.num_launches() == 1 and "rows by sizes" in t.das(), t.das()


def test_gmm_rows_past_the_last_bound_are_left_alone_and_bounds_are_clipped():
    # the last bound stops short of m: those rows keep what the buffer held; a bound past m counts as m
    m, n, k = 512, 128, 64
    x = rng(4).normal(0, 0.1, [m, k]).astype(np.float16)
    w = rng(5).normal(0, 0.1, [3, k, n]).astype(np.float16)
    t = Tester("mix")
    gl = t.load(np.array([100, 100, 400], np.int64))
    out = t.store(t.grouped_matmul(t.load(x), t.load(w), False, False, None, gl, 0))
    t.run()
    got = t.output(out)
    assert np.allclose(got[:400], gmm_split_m(x, w, None, [100, 100, 400]), rtol=1e-3, atol=1e-3)
    t.input(gl, np.array([100, 300, 9999], np.int64))   # the same program, new bounds: read on the device
    t.bare_run()
    assert np.allclose(t.output(out), gmm_split_m(x, w, None, [100, 300, 512]), rtol=1e-3, atol=1e-3)


def test_dyn_gmm_type0():  # :180-201
    t = Tester("mix:dyn")
    x, w = t.load([-1, 256], "float16"), t.load([4, 256, 2048], "float16")
    gl = t.load([-1], "int64")
    out = t.store(t.grouped_matmul(x, w, False, False, None, gl, 0))
    for x_shape, bounds in [([256, 256], [10, 100, 200, 256]), ([4096, 256], [1024, 1256, 2000, 4096])]:
        xd = Tester.fast_random_normal(0, 0.01, x_shape).astype(np.float16)
        wd = Tester.fast_random_normal(0, 0.01, [4, 256, 2048]).astype(np.float16)
        gd = np.array(bounds, np.int64)
        t.input(x, xd)
        t.input(w, wd)
        t.input(gl, gd)
        t.run()
        assert t.check(out, gmm_split_m(xd, wd, None, gd), 1e-3)


# ---- groups along k ----

@pytest.mark.parametrize("m, n, k, bounds, oracle", [
    (1024, 4096, 4096, [256, 512], False), (1024, 4096, 3333, [10, 128, 256, 1024, 2048, 3333], False), (192, 160, 333, [0, 64, 64, 200, 333], True)])
@pytest.mark.parametrize("trans", [[False, True], [True, True], [False, False], [True, False]])
def test_gmm_type2(m, n, k, bounds, trans, oracle):  # :204-229
    x = Tester.fast_random_normal(0, 0.01, [k, m] if trans[0] else [m, k]).astype(np.float16)
    w = Tester.fast_random_normal(0, 0.01, [n, k] if trans[1] else [k, n]).astype(np.float16)
    gl = np.array(bounds, np.int64)
    expect = gmm_split_k(x.T if trans[0] else x, w.T if trans[1] else w, None, gl)
    run_graph("mix", lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x), kk.load(w), trans[0], trans[1], None, kk.load(gl), 2)), expect, 1e-3)],
              oracle=oracle)


def test_gmm_type2_zero():  # :232-262 (empty groups give zeros, whatever ran before)
    t0 = Tester("mix")
    nan = np.full([1024, 1024], np.nan, np.float16)
    t0.store(t0.matmul(t0.load(nan), t0.load(nan), False, False))
    t0.run()
    m, n, k, bounds = 1024, 512, 3333, [0, 0, 10, 128, 256, 256, 1024, 2048, 2048, 3333]
    x = rng(6).normal(0, 0.01, [m, k]).astype(np.float16)
    w = rng(7).normal(0, 0.01, [k, n]).astype(np.float16)
    gl = np.array(bounds, np.int64)
    expect = gmm_split_k(x, w, None, gl)
    run_graph("mix", lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x), kk.load(w), False, False, None, kk.load(gl), 2)), expect, 1e-3)], oracle=False)


@pytest.mark.parametrize("mode", ["mix", "eager"])
@pytest.mark.parametrize("m, n, k, bounds", [(1280, 2560, 1024, [0, 256, 256, 800, 1024, 1024]), (4096, 4096, 4096, [10, 256, 3000, 4096])])
def test_gmm_type2_postfusion(mode, m, n, k, bounds):  # :265-292
    g = len(bounds)
    x = Tester.fast_random_normal(0, 0.01, [m, k]).astype(np.float16)
    w = Tester.fast_random_normal(0, 0.01, [k, n]).astype(np.float16)
    d = Tester.fast_random_normal(0, 0.01, [g, m, n]).astype(np.float32)
    gl = np.array(bounds, np.int64)
    expect = gmm_split_k(x, w, None, gl).astype(np.float16).astype(np.float32) + d

    def build(kk):
        r = kk.grouped_matmul(kk.load(x), kk.load(w), False, False, None, kk.load(gl), 2)
        return [(kk.store(kk.add(kk.load(d), kk.cast(r, "float32"))), expect, 1e-3)]

    t = run_graph(mode, build, oracle=False)
    assert t.num_launches() == 1, t.das()


def test_gmm_type2_bias_and_sizes_on_the_oracle():
    m, n, k = 130, 136, 520
    sizes = [64, 0, 200, 7, 249]
    x = rng(8).normal(0, 0.1, [m, k]).astype(np.float16)
    w = rng(9).normal(0, 0.1, [k, n]).astype(np.float16)
    bias = rng(10).normal(0, 0.1, [len(sizes), n]).astype(np.float16)
    gl = np.array(sizes, np.int64)
    expect = gmm_split_k(x, w, bias, np.cumsum(sizes))
    run_graph("mix", lambda kk: [(kk.store(kk.grouped_matmul(kk.load(x), kk.load(w), False, False, kk.load(bias), kk.load(gl), 2, 1)), expect, 2e-3)])


def test_dyn_gmm_type2():  # :295-323
    t = Tester("mix:dyn")
    x, w = t.load([4096, -1], "float16"), t.load([-1, 2048], "float16")
    z = t.load([-1, -1], "float32")
    gl = t.load([-1], "int64")
    c = t.cast(t.grouped_matmul(x, w, False, False, None, gl, 2), "float32")
    out = t.store(t.add(c, z))
    for k, bounds, z_shape in [(256, [10, 100, 200, 256], [4, 1, 2048]), (2000, [1024, 1256, 1999, 2000], [4, 1, 1]),
                               (2560, [1024, 1256, 2000, 2560], [4, 4096, 2048])]:
        xd = Tester.fast_random_normal(0, 0.1, [4096, k]).astype(np.float16)
        wd = Tester.fast_random_normal(0, 0.1, [k, 2048]).astype(np.float16)
        zd = Tester.fast_random_normal(0, 0.1, z_shape).astype(np.float32)
        gd = np.array(bounds, np.int64)
        t.input(x, xd)
        t.input(w, wd)
        t.input(z, zd)
        t.input(gl, gd)
        t.run()
        assert t.check(out, gmm_split_k(xd, wd, None, gd).astype(np.float16).astype(np.float32) + zd, 1e-3)
