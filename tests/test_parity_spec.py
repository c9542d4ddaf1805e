"""GPU parity: the reference's tests/ut/test_spec_vector.py (cited per test) through kernels created as "vector:spec"
and "vector:spec,priv1": same shapes, input distributions, NumPy expectations and tolerances. A speculative vector
kernel keeps a reduce and its consumers in one kernel where the reduced extent allows and falls back to a cut kernel
otherwise; `spec_next()` marks the stage boundaries, `priv1` lets the kernel find them. Here every kernel is compiled
that way, so what these cases probe is that the flags, the stage marker, temporary stores and bound loads are accepted
and that the graphs (reduce -> consumer, reshapes between stages, re-use of loads across stages, dynamic shapes that
fit a tile on one run and not on the next) give the reference's results."""
import numpy as np
import pytest

import dvm_amd as dvm
from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def test_spec_elemwise():  # tests/ut/test_spec_vector.py:24-31
    rng = np.random.default_rng(24)
    a0 = rng.normal(0, 1, [1024, 500]).astype(np.float32)
    t = Tester("vector:spec")
    t.store_expect(t.add(t.mul(t.load(a0), 0.1), 0.2), a0 * 0.1 + 0.2)
    assert t.run_check()


def test_spec_fall_reshape():  # :35-47
    rng = np.random.default_rng(35)
    shape_a, shape_b, shape_c, red_dims = [10, 4, 64], [10, 4, 1], [10, 32, 8], (1,)
    a = rng.normal(0.0, 0.3, shape_a).astype(np.float32)
    b = rng.normal(0.0, 0.3, shape_b).astype(np.float32)
    t = Tester("vector:spec")
    x4 = t.reshape(t.add(t.load(a), t.load(b)), shape_c)
    t.spec_next()
    t.store_expect(t.sum(x4, red_dims, True), np.sum((a + b).reshape(shape_c), axis=red_dims, keepdims=True), 1e-4)
    assert t.run_check()


@pytest.mark.parametrize("shape_a,dims", [[[2, 30, 8000], (1,)], [[4, 128], (0,)], [[3, 40], (1,)], [[500], (0,)]])
def test_spec_fall_reduce(shape_a, dims):  # :51-63
    rng = np.random.default_rng(51 + len(shape_a))
    a = rng.normal(0.0, 0.3, shape_a).astype(np.float32)
    t = Tester("vector:spec")
    x3 = t.sum(t.add(t.load(a), 0.02), dims, False)
    t.spec_next()
    x3_expect = np.sum(a + 0.02, axis=dims, keepdims=False)
    b = rng.normal(0.0, 0.3, x3_expect.shape).astype(np.float32)
    t.store_expect(t.mul(x3, t.load(b)), x3_expect * b)
    assert t.run_check()


def test_spec_migrate_load_store():  # :67-80: a value of the first stage is stored, a load of the first stage is used in the second
    rng = np.random.default_rng(67)
    a = rng.normal(0.0, 0.3, [10, 6000]).astype(np.float32)
    b = rng.normal(0.0, 0.3, [1, 6000]).astype(np.float32)
    t = Tester("vector:spec")
    x1, x2 = t.load(a), t.load(b)
    x3 = t.add(x1, 0.02)
    x4 = t.sum(x3, (0,), True)
    t.spec_next()
    x5 = t.mul(x4, x2)
    t.store_expect(x3, a + 0.02)
    t.store_expect(x5, np.sum(a + 0.02, axis=(0,), keepdims=True) * b)
    assert t.run_check()


def test_spec_load_reloc():  # :84-93: the reduced load again behind the reduce
    rng = np.random.default_rng(84)
    a = rng.normal(0.0, 0.3, [10, 6000]).astype(np.float32)
    t = Tester("vector:spec")
    x1 = t.load(a)
    x3 = t.sum(t.add(x1, 0.02), (0,), True)
    t.spec_next()
    t.store_expect(t.mul(x3, x1), np.sum(a + 0.02, axis=(0,), keepdims=True) * a)
    assert t.run_check()


def test_spec_connected_split():  # :97-109
    rng = np.random.default_rng(97)
    a = rng.normal(0.0, 0.3, [10, 6000]).astype(np.float32)
    t = Tester("vector:spec")
    x2 = t.add(t.load(a), 0.02)
    x3 = t.sum(x2, (0,), False)
    t.spec_next()
    t.store_expect(t.mul(x3, 0.5), np.sum(a + 0.02, axis=(0,), keepdims=False) * 0.5)
    t.store_expect(t.add(x2, 0.3), a + 0.02 + 0.3)
    assert t.run_check()


def test_dyn_spec_fall_reduce():  # :113-130
    rng = np.random.default_rng(113)
    t = Tester("vector:spec,dyn")
    x1 = t.load([-1], "float32")
    x2 = t.add(x1, 0.02)
    dims = t.int_array()
    x3 = t.sum(x2, dims, True)
    t.spec_next()
    x5 = t.store(t.mul(x3, x2))
    for x_shape, dims_shape in [[[3, 10, 8000], (1,)], [[100, 500], (1,)], [[8, 100], (0,)], [[4, 512], (1,)]]:
        d1 = rng.normal(0.0, 1.0, x_shape).astype(np.float32)
        t.input(x1, d1)
        dims.update(dims_shape)
        t.run()
        assert t.check(x5, np.sum(d1 + 0.02, axis=dims_shape, keepdims=True) * (d1 + 0.02), 1e-4)


def _rmsnorm_fp16(x, gamma):
    """RMSNorm in fp32 on fp16 data, the normalised value rounded to fp16 before the scale by gamma."""
    xf = x.astype(np.float32)
    return (xf / np.sqrt((xf * xf).mean(axis=1, keepdims=True) + 1e-6)).astype(np.float16) * gamma


# The case of :134-160: ONE dynamic speculative kernel object serves rows that fit a tile of the reference's vector
# core and rows that do not (65536 elements), in either order, and gets new addresses at every call. The row length
# enters the graph as an int64 scalar that is updated per call.
RELOC_SHAPES = [(2, 8192), (3, 65536), (17, 129), (4, 32768)]


@pytest.mark.parametrize("order", [RELOC_SHAPES, RELOC_SHAPES[1:] + RELOC_SHAPES[:1]], ids=["tile_first", "long_rows_first"])
def test_dyn_spec_rmsnorm_reloc(order):
    k = Tester("vector:spec,dyn")
    rows_in, scale_in, n_cols = k.load([-1, -1], "float16"), k.load([-1], "float16"), k.scalar(dvm.int64)
    v = k.cast(rows_in, "float32")
    sq = k.sum(k.mul(v, v), [1], True)
    k.spec_next()
    inv_rms = k.div(1.0, k.sqrt(k.add(k.div(sq, n_cols), 1e-6)))
    result = k.store(k.mul(k.cast(k.mul(v, inv_rms), "float16"), scale_in))
    gen = np.random.default_rng(17)
    for n_rows, width in order + order:  # every shape twice: the second visit finds the kernel object used
        data = gen.normal(0, 1, (n_rows, width)).astype(np.float16)
        gamma = gen.normal(1, 0.1, (width,)).astype(np.float16)
        k.input(rows_in, data)
        k.input(scale_in, gamma)
        n_cols.update(width)
        k.run()
        assert k.check(result, _rmsnorm_fp16(data, gamma), 3e-3), (n_rows, width)


def test_spec_dead_code():  # :164-174: a load nobody uses
    rng = np.random.default_rng(164)
    a = rng.normal(0.0, 0.3, [1024]).astype(np.float32)
    t = Tester("vector:spec", use_pass_opt=True)
    x1 = t.load(a)
    t.load(np.zeros([64], dtype=np.float32))
    x3 = t.sum(t.reshape(x1, [16, 64]), (0,), False)
    t.spec_next()
    t.store_expect(t.div(x3, 16.0), np.sum(a.reshape(16, 64), axis=0) / 16.0, 1e-4)
    assert t.run_check()


def test_auto_spec_broadcast():  # :178-189 (2000 rows instead of 10000: the graph and the row length are what matter)
    rng = np.random.default_rng(178)
    a = rng.normal(0.0, 0.3, [6000]).astype(np.float32)
    b = rng.normal(0.0, 0.3, [6000]).astype(np.float32)
    c = rng.normal(0.0, 0.3, [2000, 6000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x1 = t.add(t.load(a), t.load(b))
    x3 = t.cast(t.mul(x1, t.load(c)), "float16")
    t.store_expect(x1, a + b)
    t.store_expect(x3, ((a + b) * c).astype(np.float16))
    assert t.run_check()


@pytest.mark.parametrize("shape_a,dims", [[[2, 30, 8000], (1,)], [[3, 2, 20, 8000], (0, 2)]])
def test_auto_spec_reduce(shape_a, dims):  # :193-204
    rng = np.random.default_rng(193 + len(shape_a))
    a = rng.normal(0.0, 0.03, shape_a).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x3 = t.sum(t.add(t.load(a), 0.01), dims, True)
    x3_expect = np.sum(a + 0.01, axis=dims, keepdims=True)
    b = rng.normal(0.0, 0.3, x3_expect.shape[:-1] + (1,)).astype(np.float32)
    t.store_expect(t.mul(x3, t.load(b)), x3_expect * b)
    assert t.run_check()


def test_auto_spec_multi_reduce():  # :208-223
    rng = np.random.default_rng(208)
    a = rng.normal(0.0, 0.03, [10, 20, 1]).astype(np.float32)
    b = rng.normal(0.0, 0.03, [10, 20, 6000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x1 = t.add(t.load(a), t.load(b))
    t.store_expect(t.mul(t.sum(x1, (0,), True), 0.5), np.sum(a + b, axis=(0,), keepdims=True) * 0.5)
    x4 = t.sub(x1, 0.002)
    t.store_expect(t.add(t.sum(x4, (0,), True), 0.2), np.sum(a + b - 0.002, axis=(0,), keepdims=True) + 0.2)
    t.store_expect(t.mul(x4, 0.8), (a + b - 0.002) * 0.8)
    assert t.run_check()


def test_auto_spec_load_clone():  # :227-235
    rng = np.random.default_rng(227)
    a = rng.normal(0.0, 0.03, [4, 3, 20, 6000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x1 = t.load(a)
    x3 = t.sum(t.add(x1, 0.01), (0,), True)
    t.store_expect(t.add(x3, x1), np.sum(a + 0.01, axis=(0,), keepdims=True) + a)
    assert t.run_check()


def test_auto_spec_nest_reduce():  # :239-251
    rng = np.random.default_rng(239)
    a = rng.normal(0.0, 0.03, [4, 3, 20, 1]).astype(np.float32)
    b = rng.normal(0.0, 0.03, [4, 3, 20, 6000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x3 = t.mul(t.sum(t.add(t.load(a), t.load(b)), (2,), True), 0.5)
    x5 = t.add(t.sum(x3, (0,), True), x3)
    e3 = np.sum(a + b, axis=(2,), keepdims=True) * 0.5
    t.store_expect(x5, np.sum(e3, axis=(0,), keepdims=True) + e3)
    assert t.run_check()


@pytest.mark.parametrize("shape1,shape2,shape3,red_dims", [
    [[1, 2000], [20, 2000], [20 * 2000], (0,)],
    [[10, 200], [10, 200], [5, 10, 40], (2,)],
    [[10, 1], [1, 200], [5, 10, 40], (1,)],
])
def test_auto_spec_reshape_reduce(shape1, shape2, shape3, red_dims):  # :255-272: (a + b).reshape(shape3).sum(red_dims)
    rng = np.random.default_rng(255 + len(shape3))
    a = rng.normal(0.0, 0.03, shape1).astype(np.float32)
    b = rng.normal(0.0, 0.03, shape2).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x3 = t.sum(t.reshape(t.add(t.load(a), t.load(b)), shape3), red_dims, True)
    x4 = t.mul(x3, 0.8)
    x5 = t.add(x4, x3)
    e3 = np.sum((a + b).reshape(shape3), axis=red_dims, keepdims=True)
    t.store_expect(x4, e3 * 0.8)
    t.store_expect(x5, (e3 * 0.8) + e3)
    assert t.run_check()


def test_auto_spec_reshape_chains():  # :276-311: reshapes between pointwise stages, back to back, eliminated
    rng = np.random.default_rng(276)
    a = rng.normal(0.0, 0.03, [10, 1000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x3 = t.mul(t.reshape(t.add(t.load(a), 0.01), [10000]), 0.7)
    t.store_expect(t.add(t.reshape(x3, [20, 500]), 0.2), ((a + 0.01).reshape([10000]) * 0.7).reshape([20, 500]) + 0.2)
    assert t.run_check()
    t = Tester("vector:spec,priv1")
    x3 = t.mul(t.reshape(t.add(t.load(a), 0.01), [10000]), 0.7)
    t.store_expect(t.sub(t.reshape(x3, [50, 200]), 0.01), ((a + 0.01).reshape([10000]) * 0.7).reshape([50, 200]) - 0.01)
    assert t.run_check()
    t = Tester("vector:spec,priv1")
    x3 = t.reshape(t.reshape(t.add(t.load(a), 0.01), [10000]), [20, 500])
    t.store_expect(t.add(x3, 0.2), (a + 0.01).reshape([20, 500]) + 0.2)
    assert t.run_check()


def test_auto_spec_reshape_cross_dim():  # :315-323
    rng = np.random.default_rng(315)
    a = rng.normal(0.0, 0.03, [10, 1000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x0 = t.load(a)
    t.store_expect(t.add(t.reshape(x0, [1, 10, 1000]), t.reshape(x0, [10, 1, 1000])), a.reshape([1, 10, 1000]) + a.reshape([10, 1, 1000]))
    assert t.run_check()


def test_auto_spec_reshape_side_connect():  # :327-336
    rng = np.random.default_rng(327)
    a = rng.normal(0.0, 0.03, [10, 1, 1000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x1 = t.add(t.load(a), 0.1)
    t.store_expect(t.mul(t.reshape(x1, [1, 10, 1000]), x1), (a + 0.1).reshape([1, 10, 1000]) * (a + 0.1))
    assert t.run_check()


def test_auto_spec_dyn_shape():  # :340-362 (both inputs take x_shape there too)
    rng = np.random.default_rng(340)
    t = Tester("vector:spec,dyn,priv1")
    x1, x2 = t.load([-1], "float32"), t.load([-1], "float32")
    x3 = t.add(x1, x2)
    x4 = t.store(t.mul(x3, 1.2))
    dims = t.int_array()
    x7 = t.store(t.mul(t.sum(x3, dims, True), 0.01))
    for x_shape, dims_shape in [[[30, 8000], (0,)], [[512, 1000], (1,)], [[4, 1000, 1], (1,)], [[10, 1, 20, 512], (0, 3)]]:
        d1 = rng.normal(0.0, 1.0, x_shape).astype(np.float32)
        d2 = rng.normal(0.0, 1.0, x_shape).astype(np.float32)
        t.input(x1, d1)
        t.input(x2, d2)
        dims.update(dims_shape)
        t.run()
        assert t.check(x4, (d1 + d2) * 1.2)
        assert t.check(x7, np.sum(d1 + d2, axis=dims_shape, keepdims=True) * 0.01, 1e-4)


@pytest.mark.parametrize("mode", ["vector:spec", "vector:spec,priv1"])
def test_spec_swap_with_store(mode):  # :366-380: the reduce result is stored and used by the next stage
    rng = np.random.default_rng(366)
    shape_a, dims = [2, 30, 8000], (1,)
    a = rng.normal(0.0, 0.03, shape_a).astype(np.float32)
    t = Tester(mode)
    x3 = t.sum(t.add(t.load(a), 0.01), dims, True)
    x3_expect = np.sum(a + 0.01, axis=dims, keepdims=True)
    t.store_expect(x3, x3_expect, 1e-4)
    t.spec_next()
    b = rng.normal(0.0, 0.3, x3_expect.shape[:-1] + (1,)).astype(np.float32)
    t.store_expect(t.mul(x3, t.load(b)), x3_expect * b, 1e-4)
    assert t.run_check()


def test_auto_spec_indirect_cut_depend():  # :384-397
    rng = np.random.default_rng(384)
    a = rng.normal(0.0, 0.03, [4, 3, 20, 1]).astype(np.float32)
    b = rng.normal(0.0, 0.03, [4, 3, 20, 6000]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x1 = t.add(t.load(a), t.load(b))
    x3 = t.mul(t.sum(x1, (0,), True), 0.5)
    x4 = t.add(x3, x1)
    e3 = np.sum(a + b, axis=(0,), keepdims=True) * 0.5
    t.store_expect(x3, e3)
    t.store_expect(x4, e3 + (a + b))
    assert t.run_check()


def test_spec_custom():  # :401-412: a temporary store and a load bound to it hand a value on inside the kernel
    rng = np.random.default_rng(401)
    a0 = rng.normal(0, 1, [1024, 500]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x1 = t.store(t.mul(t.load(a0), 0.1))
    x2 = t.load([1024, 500], "float32")
    t.set_store_temp(x1)
    t.set_load_bind(x2, x1)
    t.store_expect(t.add(x2, 0.2), a0 * 0.1 + 0.2)
    assert t.run_check()
    assert t.num_launches() == 1, t.das()


def test_a_bound_load_of_a_store_that_stays_an_output():
    # without set_store_temp the store is still written; binding after the load's first use is refused
    rng = np.random.default_rng(402)
    a0 = rng.normal(0, 1, [64, 500]).astype(np.float32)
    t = Tester("vector")
    x1 = t.store_expect(t.mul(t.load(a0), 0.1), a0 * np.float32(0.1))
    x2 = t.load([64, 500], "float32")
    t.set_load_bind(x2, x1)
    t.store_expect(t.sum(t.add(x2, 0.2), (1,), True), np.sum(a0 * np.float32(0.1) + 0.2, axis=1, keepdims=True), 1e-4)
    assert t.run_check()
    t = Tester("vector")
    x1 = t.store(t.mul(t.load(a0), 0.1))
    x2 = t.load([64, 500], "float32")
    t.add(x2, 0.2)
    with pytest.raises(RuntimeError, match="before the first use"):
        t.set_load_bind(x2, x1)
    with pytest.raises(RuntimeError, match="kSpeculate"):
        Tester("vector").spec_next()


@pytest.mark.parametrize("is_split", [True, False])
def test_spec_slice(is_split):  # :416-427
    rng = np.random.default_rng(416)
    a0 = rng.normal(0, 1, [1024, 500]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x0 = t.load(a0)
    if is_split:
        x0 = t.mul(x0, 0.1)
        a0 = a0 * np.float32(0.1)
    t.store_expect(t.add(t.slice(x0, [100, 100], [600, 300]), 0.2), a0[100:700, 100:400] + 0.2)
    assert t.run_check()


@pytest.mark.parametrize("is_split,end", [[True, 700], [True, -2], [False, 100000]])
def test_spec_slice_dim(is_split, end):  # :431-445
    rng = np.random.default_rng(431)
    a0 = rng.normal(0, 1, [1024, 500]).astype(np.float32)
    t = Tester("vector:spec,priv1")
    x0 = t.load(a0)
    if is_split:
        x0 = t.mul(x0, 0.1)
        a0 = a0 * np.float32(0.1)
    b_ref = t.scalar(dvm.int64)
    b_ref.update(100)
    t.store_expect(t.add(t.slice_dim(x0, 0, b_ref, end), 0.2), a0[100:end, :] + 0.2)
    assert t.run_check()
