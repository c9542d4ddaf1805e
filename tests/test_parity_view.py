"""GPU parity: strided views, restating tests/ut/test_view.py and tests/ut/test_slice.py of the reference (cited
per test): loads that read part of a buffer through a stride list (slices, strided columns, transposes, zero
strides, an element offset), slice loads with start/size or start/end/step, and stores that write through a
stride list into a larger, zero-filled buffer. Same shapes, strides and NumPy expectations as there; every graph
also runs on the CPU oracle. The reference's `tile(...)` calls pick a loop split of its own code generator and
do not change results, so they have no counterpart here."""
import numpy as np
import pytest

from tests.util import run_graph

pytestmark = pytest.mark.gpu


def rng(seed=0):
    return np.random.default_rng(seed)


def row_major(shape):
    st = [1] * len(shape)
    for i in range(len(shape) - 1, 0, -1):
        st[i - 1] = st[i] * shape[i]
    return st


def crop(a, shape):
    return a[tuple(slice(0, n) for n in shape)]


# ---- strided loads ----

@pytest.mark.parametrize("in_shape, slice_shape", [([30, 1000], [20, 500]), ([30, 500], [20, 200]),
                                                   ([30, 4000], [20, 3000]), ([43, 1000], [40, 500])])
def test_slice_2d(in_shape, slice_shape):  # tests/ut/test_view.py:40-60
    a = rng(1).normal(0, 1, in_shape).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load(slice_shape, row_major(in_shape), a), 0.1)),
                              crop(a, slice_shape) + np.float32(0.1), None)])


@pytest.mark.parametrize("in_shape, slice_shape", [
    ([24, 20, 100], [20, 10, 60]), ([24, 20, 1000], [20, 10, 600]), ([24, 20, 1000], [20, 20, 600]),
    ([24, 20, 64], [20, 15, 64]), ([24, 15, 64], [20, 15, 64]), ([200, 20, 100], [200, 20, 30]),
    ([200, 20, 60], [200, 10, 30]), ([200, 20, 20], [200, 10, 20])])
def test_slice_3d(in_shape, slice_shape):  # :63-93
    a = rng(2).normal(0, 1, in_shape).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load(slice_shape, row_major(in_shape), a), 0.1)),
                              crop(a, slice_shape) + np.float32(0.1), None)])


@pytest.mark.parametrize("in_shape, slice_shape", [([4, 4, 5, 3, 16], [3, 2, 3, 2, 12]),
                                                   ([4, 4, 4, 5, 6, 16], [3, 2, 3, 4, 5, 12])])
def test_slice_loop(in_shape, slice_shape):  # :96-121 (five and six dimensions, none of them mergeable)
    a = rng(3).normal(0, 1, in_shape).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load(slice_shape, row_major(in_shape), a), 0.1)),
                              crop(a, slice_shape) + np.float32(0.1), None)])


def test_slice_dim_fold():  # :124-134
    a = rng(4).normal(0, 1, [4, 2, 64, 96]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load([4, 2, 64, 64], [12288, 6144, 96, 1], a), 0.1)),
                              a[:, :, :, 0:64] + np.float32(0.1), None)])


def test_slice_dim_x():  # :137-144 (every tenth column)
    a = rng(5).normal(0, 1, [100, 2048]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load([100, 200], [2048, 10], a), 0.1)),
                              a[:, 0:2000:10] + np.float32(0.1), None)])


def test_slice_dim_x_fp16_large():  # :147-154 (the reference's [4096, 20000] at a quarter of the rows)
    a = rng(6).normal(0, 1, [1024, 20000]).astype(np.float16)
    run_graph("", lambda k: [(k.store(k.add(k.view_load([1024, 10000], [20000, 2], a), 0.1)),
                              a[:, 0:20000:2] + np.float16(0.1), 1e-3)])


def test_slice_dim_x_lead_1():  # :157-164
    a = rng(7).normal(0, 1, [100, 2048, 1]).astype(np.float16)
    run_graph("", lambda k: [(k.store(k.add(k.view_load([100, 199, 1], [2048, 10, 1], a), 0.1)),
                              a[:, 0:1990:10, :] + np.float16(0.1), 1e-3)])


@pytest.mark.parametrize("stride_elem", [2, 3, 4, 5, 6, 7, 8])
def test_slice_dim_x_stride(stride_elem):  # :167-180
    shape = [8, 64]
    in_shape = [shape[0], shape[1] * stride_elem]
    row = ((np.arange(in_shape[0], dtype=np.float32) % 251) * 0.01).astype(np.float16)
    col = ((np.arange(in_shape[1], dtype=np.float32) % 257) * 0.001).astype(np.float16)
    a = (row[:, None] + col[None, :]).astype(np.float16, copy=False)
    run_graph("", lambda k: [(k.store(k.add(k.view_load(shape, [in_shape[1], stride_elem], a), 0.5)),
                              a[:, 0:shape[1] * stride_elem:stride_elem] + np.float16(0.5), 1e-3)])


@pytest.mark.parametrize("shape, dim0, dim1", [([8, 30, 512], 0, 1), ([8, 6, 20, 64], 1, 2), ([8, 6, 20, 64], 0, 2),
                                               ([1024, 512], 0, 1)])
def test_transpose(shape, dim0, dim1):  # :183-201
    a = rng(8).normal(0, 1, shape).astype(np.float32)
    vshape, stride = list(shape), row_major(shape)
    vshape[dim0], vshape[dim1] = vshape[dim1], vshape[dim0]
    stride[dim0], stride[dim1] = stride[dim1], stride[dim0]
    run_graph("", lambda k: [(k.store(k.add(k.view_load(vshape, stride, a), 0.1)),
                              np.swapaxes(a, dim0, dim1) + np.float32(0.1), None)])


@pytest.mark.parametrize("shape, new_shape", [([1, 10, 64], [40, 10, 64]), ([1, 1, 64], [40, 10, 64]),
                                              ([1, 3, 1, 64], [5, 3, 10, 64]), ([8, 1, 1, 1], [8, 3, 10, 64])])
def test_broadcast(shape, new_shape):  # :204-222 (zero strides)
    a = rng(9).normal(0, 1, shape).astype(np.float32)
    stride, cur = [1] * len(shape), 1
    for i in range(len(shape) - 1, -1, -1):
        stride[i] = 0 if shape[i] != new_shape[i] else cur
        cur *= shape[i]
    run_graph("", lambda k: [(k.store(k.add(k.view_load(new_shape, stride, a), 0.1)),
                              np.broadcast_to(a, new_shape) + np.float32(0.1), None)])


def test_broadcast_of_slice_six_dims():  # :225-243
    shape, sshape, bshape = [1, 10, 1, 20, 8, 32], [1, 6, 1, 18, 7, 32], [4, 6, 8, 18, 7, 32]
    a = rng(10).normal(0, 1, shape).astype(np.float32)
    b = rng(11).normal(0, 1, bshape).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load(sshape, row_major(shape), a), k.load(b))),
                              a[:, :6, :, :18, :7, :] + b, None)])


def test_view_lead_strided_column():  # :246-255
    a = rng(12).normal(0, 0.1, [32, 1, 1, 1]).astype(np.float32)
    b = rng(13).normal(0, 0.1, [16, 10, 1, 4000]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.view_load([16, 1, 1, 1], [2, 1, 1, 1], a), k.load(b))),
                              a[::2, :, :, :] + b, None)])


@pytest.mark.parametrize("shape, split_dim, split_num, split_idx", [([40, 100, 64], 1, 5, 3), ([40, 1000], 1, 5, 0)])
def test_split(shape, split_dim, split_num, split_idx):  # :258-279 (an element offset into the buffer)
    a = rng(14).normal(0, 1, shape).astype(np.float32)
    size = shape[split_dim] // split_num
    new_shape = [n if i != split_dim else size for i, n in enumerate(shape)]
    stride = row_major(shape)
    offset = split_idx * size * stride[split_dim]
    run_graph("", lambda k: [(k.store(k.add(k.view_load(new_shape, stride, a, offset), 0.1)),
                              np.split(a, split_num, split_dim)[split_idx] + np.float32(0.1), None)])


@pytest.mark.parametrize("slice_shape, in_shape, broadcast_shape", [([3, 30, 100], [3, 60, 200], [4, 3, 30, 100]),
                                                                    ([4, 1, 512], [6, 2, 512], [4, 8, 512])])
def test_view_load_broadcast_3d(slice_shape, in_shape, broadcast_shape):  # :282-295
    a = rng(15).normal(0, 1, in_shape).astype(np.float32)
    b = rng(16).normal(0, 1, broadcast_shape).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.add(k.add(k.view_load(slice_shape, row_major(in_shape), a), 0.1), k.load(b))),
                              crop(a, slice_shape) + np.float32(0.1) + b, None)])


def test_view_load_zero_strides_in_the_middle():  # :298-313
    a = rng(17).normal(0, 1, [4, 512]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.view_load([4, 5, 500, 512], [512, 0, 0, 1], a)),
                              np.broadcast_to(a[:, None, None, :], (4, 5, 500, 512)), 0)])
    run_graph("", lambda k: [(k.store(k.view_load([4, 5, 500, 128], [512, 0, 0, 4], a)),
                              np.broadcast_to(a[:, None, None, :512:4], (4, 5, 500, 128)), 0)])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_view_load_many_strides_in_one_kernel(dtype):  # :476-496
    rows, width = 65, 17
    r = rng(42)
    datas = [(s, r.uniform(-1, 1, size=(rows, 4, width * s)).astype(dtype)) for s in [2, 3, 5, 6, 8, 4, 7, 3]]
    expected = sum(d[..., ::s].transpose(1, 0, 2).astype(np.float32) for s, d in datas)

    def g(k):
        acc = None
        for s, d in datas:
            x = k.cast(k.view_load([4, rows, width], [width * s, 4 * width * s, s], d), "float32")
            acc = x if acc is None else k.add(acc, x)
        return [(k.store(acc), expected, 1e-6)]
    run_graph("vector", g)


# ---- strided stores ----

def padded(shape, value):
    e = np.zeros(shape, value.dtype)
    e[tuple(slice(0, n) for n in value.shape)] = value
    return e


@pytest.mark.parametrize("out_shape, slice_shape", [([30, 1000], [20, 500]), ([30, 500], [20, 200]),
                                                    ([30, 4000], [20, 3000]), ([43, 1000], [40, 500])])
def test_view_store_2d(out_shape, slice_shape):  # :316-338
    a = rng(20).normal(0, 1, slice_shape).astype(np.float32)
    e = padded(out_shape, a + np.float32(0.1))
    run_graph("", lambda k: [(k.view_store_expect(k.add(k.load(a), 0.1), row_major(out_shape), e), e, None)])


@pytest.mark.parametrize("out_shape, slice_shape", [
    ([24, 20, 100], [20, 10, 60]), ([24, 20, 1000], [20, 10, 600]), ([24, 20, 1000], [20, 20, 600]),
    ([24, 20, 64], [20, 15, 64]), ([24, 15, 64], [20, 15, 64]), ([200, 20, 100], [200, 20, 30]),
    ([200, 20, 60], [200, 10, 30]), ([200, 20, 20], [200, 10, 20]),
    ([4, 4, 5, 3, 16], [3, 2, 3, 2, 12]), ([4, 4, 4, 5, 6, 16], [3, 2, 3, 4, 5, 12]), ([4, 2, 64, 96], [4, 2, 64, 64])])
def test_view_store_nd(out_shape, slice_shape):  # :341-411
    a = rng(21).normal(0, 1, slice_shape).astype(np.float32)
    e = padded(out_shape, a + np.float32(0.1))
    run_graph("", lambda k: [(k.view_store_expect(k.add(k.load(a), 0.1), row_major(out_shape), e), e, None)])


@pytest.mark.parametrize("slice_shape, out_shape, broadcast_shape", [([3, 30, 100], [3, 60, 200], [4, 3, 30, 100]),
                                                                     ([4, 1, 512], [6, 2, 512], [4, 8, 512])])
def test_view_store_broadcast_3d(slice_shape, out_shape, broadcast_shape):  # :414-429
    a = rng(22).normal(0, 1, slice_shape).astype(np.float32)
    b = rng(23).normal(0, 1, broadcast_shape).astype(np.float32)
    e = padded(out_shape, a + np.float32(0.1))

    def g(k):
        x0 = k.add(k.load(a), 0.1)
        s0 = k.view_store_expect(x0, row_major(out_shape), e)
        return [(s0, e, None), (k.store(k.add(x0, k.load(b))), a + np.float32(0.1) + b, None)]
    run_graph("", g)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_view_store_every_third_column(dtype):  # :432-441
    a = rng(24).normal(0, 1, [400, 600]).astype(dtype)
    e = np.zeros([400, 2000], dtype)
    e[:, :1800:3] = a + dtype(0.1)
    run_graph("", lambda k: [(k.view_store_expect(k.add(k.load(a), 0.1), [2000, 3], e), e, 1e-3 if dtype == np.float16 else None)])


def test_view_store_transpose():  # :444-449
    a = rng(25).normal(0, 1, [2000, 4000]).astype(np.float32)
    e = np.ascontiguousarray(np.swapaxes(a, 0, 1))
    run_graph("", lambda k: [(k.view_store_expect(k.load(a), [1, 2000], e), e, 0)])


@pytest.mark.parametrize("in_shape, dims, out_shape", [([100, 1000], (0,), [100, 1200]), ([10, 16, 1000], (1,), [10, 18, 1100]),
                                                       ([20, 8, 1000], (0,), [20, 10, 1200]),
                                                       ([10, 8, 12, 1000], (0, 2), [10, 10, 16, 1000])])
def test_view_store_of_a_reduce(in_shape, dims, out_shape):  # :452-473
    a = rng(26).normal(-0.5, 0.5, in_shape).astype(np.float32)
    e = padded(out_shape, np.sum(a, dims, keepdims=True))
    run_graph("", lambda k: [(k.view_store_expect(k.sum(k.load(a), dims, True), row_major(out_shape), e), e, 1e-4)])


# ---- slice loads, tests/ut/test_slice.py ----

@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("shape, start, size", [((32, 32), (3, 3), (16, 16)), ((32, 32), (3, 3), (8, 13)), ((4, 4097), (0, 0), (2, 4097)),
                                                ((111, 111), (22, 22), (33, 33)), ((16, 4096), (4, 222), (3, 332))])
def test_slice_load_2d(dtype, shape, start, size):  # tests/ut/test_slice.py:8-22 (shapes in the style of its 1-D and 3-D lists)
    a = rng(30).normal(0, 1, shape).astype(dtype)
    g = np.exp(a[start[0]:start[0] + size[0], start[1]:start[1] + size[1]])
    run_graph("", lambda k: [(k.store(k.exp(k.slice_load(a, start, size))), g, 1e-3 if dtype == np.float16 else None)])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("shape, start, size", [((32,), (3,), (16,)), ((32,), (3,), (8,)), ((4,), (0,), (2,)),
                                                ((1111,), (222,), (333,)), ((1621,), (4,), (333,))])
def test_slice_load_1d(dtype, shape, start, size):  # :25-38
    a = rng(31).normal(0, 1, shape).astype(dtype)
    g = np.exp(a[start[0]:start[0] + size[0]])
    eps = 1e-3 if dtype == np.float16 else None
    run_graph("", lambda k: [(k.store(k.exp(k.slice_load(a, start, size))), g, eps)])
    run_graph("", lambda k: [(k.store(k.exp(k.stridedslice_load(a, start, (start[0] + size[0],), (1,)))), g, eps)])  # :41-54


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("shape, start, size", [((32, 32, 4), (3, 3, 1), (16, 16, 2)), ((32, 32, 10), (3, 3, 1), (8, 13, 8)),
                                                ((4, 4097, 20), (0, 0, 5), (2, 4097, 5)), ((111, 111, 111), (22, 22, 22), (33, 33, 32)),
                                                ((16, 11, 4096), (4, 4, 222), (3, 3, 332)), ((32, 33, 34), (3, 5, 7), (27, 6, 5))])
def test_slice_load_3d(dtype, shape, start, size):  # :57-73
    a = rng(32).normal(0, 1, shape).astype(dtype)
    g = dtype(2) * a[tuple(slice(s, s + n) for s, n in zip(start, size))]
    run_graph("", lambda k: [(k.store(k.mul(k.slice_load(a, start, size), 2)), g, 0)])


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int32])
@pytest.mark.parametrize("shape, start, end", [((32, 32, 4), 1, -2), ((32, 7, 7), -30, 12), ((32, 7, 7), -30, 100), ((14, 4097, 20), -4, -1)])
def test_slice_start_end(dtype, shape, start, end):  # :76-89 (negative and out-of-range bounds)
    a = rng(33).normal(0, 1, shape).astype(dtype)
    g = dtype(2) * a[start:end]
    run_graph("", lambda k: [(k.store(k.mul(k.stridedslice_load(a, (start, 0, 0), (end, shape[1], shape[2]), (1, 1, 1)), 2)), g, 0)])


def test_strided_slice_steps():  # steps above one, which the reference's StridedSliceLoad takes (include/dvm.h:317)
    a = rng(34).normal(0, 1, (40, 9, 70)).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.mul(k.stridedslice_load(a, (1, 0, 2), (38, 9, 64), (3, 2, 1)), 2)), np.float32(2) * a[1:38:3, 0:9:2, 2:64], 0)])
    run_graph("", lambda k: [(k.store(k.mul(k.stridedslice_load(a, (0, 1, 1), (40, 8, 70), (1, 1, 4)), 2)), np.float32(2) * a[:, 1:8, 1:70:4], 0)])


def test_slice_broadcast():  # :92-101
    a = rng(35).normal(0, 1, [1, 10, 20, 30]).astype(np.float32)
    b = rng(36).normal(0, 1, [10, 10, 20, 1]).astype(np.float32)
    run_graph("", lambda k: [(k.store(k.mul(k.slice_load(a, (0, 0, 0, 0), (1, 10, 20, 15)), k.load(b))), a[:, :, :, 0:15] * b, None)])


def test_slice_mixed_with_casts():  # :104-123 (the reference's [1, 14, 41850, 40] with 4185 rows)
    n = 4185
    a = rng(37).normal(0, 1, (1, 14, n, 40)).astype(np.float16)
    b = rng(38).normal(0, 1, (2, 1, n, 80)).astype(np.float16)
    c = rng(39).normal(0, 1, (1, 14, n, 40)).astype(np.float16)
    g = (a.astype(np.float32) * b[:, :, :, 0:40].astype(np.float32) + c.astype(np.float32)).astype(np.float16)

    def build(k):
        x = k.cast(k.load(a), "float32")
        y = k.cast(k.slice_load(b, (0, 0, 0, 0), (2, 1, n, 40)), "float32")
        z = k.add(k.cast(k.load(c), "float32"), k.mul(x, y))
        return [(k.store(k.cast(z, "float16")), g, 1e-3)]
    run_graph("", build)


# ---- transposes read through strides, tests/ut/test_view_sch.py:22-106, 221-243, 777-785 (the kernel flag there picks the
# reference's fractal transpose; the tile counts in its comments are its own) ----

@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("h,w", [(1024, 2048), (38, 1024), (1024, 38), (100, 70), (2000, 900), (300, 10), (7, 300), (7, 12)])
def test_transpose_through_a_strided_load_and_a_strided_store(dtype, h, w):
    a = rng(h + w).normal(0, 1, (w, h)).astype(dtype)
    e = np.ascontiguousarray(a.T)
    run_graph("vector:opt_fractal", lambda k: [(k.view_store_expect(k.view_load([h, w], [1, h], a), [w, 1], e), e, 0)])


@pytest.mark.parametrize("shape1,swap1,shape2,swap2,strided_store", [
    ([10, 64, 200], (1, 2), [10, 64, 200], (1, 2), True), ([4, 70, 20, 200], (1, 3), [1, 70, 20, 200], (1, 3), False),
    ([10, 1, 200], (1, 2), [10, 128, 200], (1, 2), True), ([10, 200, 1], (1, 2), [10, 200, 128], (1, 2), False),
    ([5, 3, 32, 1], (2, 3), [5, 3, 32, 129], (2, 3), True)])
def test_sum_of_two_transposing_loads(shape1, swap1, shape2, swap2, strided_store):
    a, b = rng(31).normal(0, 1, shape1).astype(np.float32), rng(32).normal(0, 1, shape2).astype(np.float32)
    ta, tb = np.swapaxes(a, *swap1), np.swapaxes(b, *swap2)
    s1, s2 = row_major(shape1), row_major(shape2)
    s1[swap1[0]], s1[swap1[1]] = s1[swap1[1]], s1[swap1[0]]
    s2[swap2[0]], s2[swap2[1]] = s2[swap2[1]], s2[swap2[0]]
    e = np.ascontiguousarray(ta + tb)

    def g(k):
        v = k.add(k.view_load(list(ta.shape), s1, a), k.view_load(list(tb.shape), s2, b))
        return [(k.view_store_expect(v, row_major(list(e.shape)), e) if strided_store else k.store(v), e, 0)]
    run_graph("vector:opt_fractal", g)


def test_transposed_column_plus_transposed_rows_of_23():
    lhs = rng(33).normal(0, 1, [1, 1, 2, 1]).astype(np.float16)
    rhs = rng(34).normal(0, 1, [4, 1, 23, 257]).astype(np.float16)
    e = np.swapaxes(lhs, 1, 2) + np.swapaxes(rhs, 2, 3)

    def g(k):
        x = k.view_load([1, 2, 1, 1], [2, 1, 2, 1], lhs)
        y = k.view_load([4, 1, 257, 23], [5911, 5911, 1, 257], rhs)
        return [(k.store(k.copy(k.add(x, y))), e, 0)]
    run_graph("", g)


@pytest.mark.parametrize("shape,swap", [([4, 70, 20, 200], (1, 3)), ([2, 2048, 16, 128], (2, 3)), ([129, 128], (0, 1))])
def test_transpose_of_two_axes_of_a_larger_tensor(shape, swap):
    a = rng(35).normal(0, 1, shape).astype(np.float16)
    e = np.ascontiguousarray(np.swapaxes(a, *swap))
    s = row_major(shape)
    s[swap[0]], s[swap[1]] = s[swap[1]], s[swap[0]]
    run_graph("vector:opt_fractal", lambda k: [(k.view_store_expect(k.view_load(list(e.shape), s, a), row_major(list(e.shape)), e), e, 0)])


@pytest.mark.parametrize("shape1,shape2", [([3, 18911], [3, 1]), ([2, 18911, 3], [2, 1, 3]), ([3, 15401, 3], [3, 1, 1])])
@pytest.mark.parametrize("through_strides", [True, False])
def test_long_odd_rows_plus_a_broadcast_operand(shape1, shape2, through_strides):
    a, b = rng(36).normal(0, 1, shape1).astype(np.float32), rng(37).normal(0, 1, shape2).astype(np.float32)
    e = a + b

    def g(k):
        if through_strides:
            v = k.add(k.view_load(shape1, row_major(shape1), a), k.view_load(shape2, row_major(shape2), b))
            return [(k.view_store_expect(v, row_major(list(e.shape)), e), e, 0)]
        return [(k.store(k.add(k.load(a), k.load(b))), e, 0)]
    run_graph("", g)


def test_split_and_slice_of_a_load_with_gaps_meet_again():
    a0 = np.arange(64, dtype=np.float32).reshape(8, 8)

    def g(k):
        vl = k.view_load([8, 4], [8, 2], a0)
        _, second = k.split(vl, 1, 2, 2)
        return [(k.store(k.add(second, k.slice(vl, [0, 2], [8, 2]))), 2 * a0[:, [4, 6]], 0)]
    run_graph("", g)
