"""GPU parity: attention. The graph of examples/03_attention.py runs as three sub-kernels when the
fused kernel does not apply, as one fused launch when it does; both against the example's NumPy
golden (1e-2), the unfused one also against the CPU oracle."""
import math

import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_parity

pytestmark = pytest.mark.gpu


def np_attention(q, k, v):  # examples/03_attention.py:20-28, batched
    scale = 1.0 / math.sqrt(q.shape[-1])
    s = np.matmul(q.astype(np.float32), np.swapaxes(k.astype(np.float32), -1, -2)) * scale
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(-1, keepdims=True)
    return np.matmul(p, v.astype(np.float32))


def attention_graph(k, q, kk, v, scale, rank, dt="float16"):  # examples/03_attention.py:30-50
    s = k.mul(k.matmul(q, kk, False, True), scale)
    x = k.cast(s, "float32")
    x = k.sub(x, k.max(x, (rank - 1,), True))
    e = k.exp(x)
    p = k.cast(k.div(e, k.sum(e, (rank - 1,), True)), dt)
    return k.matmul(p, v, False, False)


def _bf16(x):
    return Tester.convert_from_bf16(Tester.convert_to_bf16(x.astype(np.float32)))


def test_attention_example_small():  # examples/03_attention.py:52-63: too small for the fused kernel
    rng = np.random.default_rng(0)
    q, k, v = (rng.normal(0, 0.02, s).astype(np.float16) for s in ((4, 8), (6, 8), (6, 12)))
    run_parity(lambda kk, a, b, c: attention_graph(kk, a, b, c, 1.0 / math.sqrt(8), 2), [q, k, v], ker="mix",
               golden=np_attention(q, k, v).astype(np.float16), eps=1e-2)


def _fused(q, k, v, dt="float16"):
    t = Tester("mix")
    dts = dt if dt == "bfloat16" else None
    out = t.store(attention_graph(t, t.load(q, dts), t.load(k, dts), t.load(v, dts), 1.0 / math.sqrt(q.shape[-1]), q.ndim, dt))
    t.run()
    assert "entry attention" in t.das() and t.num_launches() == 1, t.das()
    o = t.output(out)
    return Tester.convert_from_bf16(o) if dt == "bfloat16" else o


@pytest.mark.parametrize("waves", ["8", "4"])  # the kernel has a build on eight waves (the default) and one on four
@pytest.mark.parametrize("shape", [((2, 3), 256, 192), ((1,), 64, 64), ((3,), 100, 128), ((2, 2), 300, 2048), ((), 513, 640)])
@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
def test_attention_fused(monkeypatch, shape, dt, waves):
    monkeypatch.setenv("DVM_ATTN_WAVES", waves)
    batch, sq, skv = shape
    rng = np.random.default_rng(sq)
    conv = (lambda x: x.astype(np.float16)) if dt == "float16" else _bf16
    q, k, v = (conv(rng.standard_normal(batch + (n, 128))) for n in (sq, skv, skv))
    got = _fused(q, k, v, dt)
    want = np_attention(q, k, v)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-2, atol=1e-2), np.abs(got - want).max()


@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
@pytest.mark.parametrize("spread,d", [(20.0, 128), (20.0, 64), (0.0, 128), (6.0, 64)])
def test_attention_sharp_and_flat_softmax(dt, spread, d):
    # scores hundreds apart (the weights of a row are one key's, the rest underflow) and scores all equal
    rng = np.random.default_rng(int(spread) + d)
    conv = (lambda x: x.astype(np.float16)) if dt == "float16" else _bf16
    q, k, v = (conv(rng.standard_normal((2, n, d)) * s) for n, s in ((300, spread), (520, spread), (520, 1.0)))
    if spread > 0:
        k[:, 7, :] = q[:, 0, :]  # query 0 has one key far above the rest
    got, want = _fused(q, k, v, dt), np_attention(q, k, v)
    assert not np.isnan(got).any()
    assert np.allclose(got, want, rtol=2e-2, atol=2e-2), np.abs(got - want).max()


def test_attention_fused_constant_values_and_key_order():
    # softmax weights sum to one: with every row of V equal to c the output rows are c, at any size;
    # and the result does not depend on the order of the keys
    rng = np.random.default_rng(5)
    q, k = (rng.standard_normal((4, 512, 128)).astype(np.float16) for _ in range(2))
    c = rng.standard_normal(128).astype(np.float16)
    got = _fused(q, k, np.broadcast_to(c, (4, 512, 128)).copy())
    assert np.allclose(got, c, rtol=2e-3, atol=2e-3)
    v = rng.standard_normal((4, 512, 128)).astype(np.float16)
    perm = rng.permutation(512)
    a, b = _fused(q, k, v), _fused(q, k[:, perm], v[:, perm])
    assert np.allclose(a, b, rtol=5e-3, atol=5e-3)


def test_attention_full_size_heads():  # BASELINE config 4 shape, three sampled heads against the golden
    rng = np.random.default_rng(1004)
    q, k, v = (rng.standard_normal((8, 32, 2048, 128), dtype=np.float32).astype(np.float16) for _ in range(3))
    got = _fused(q, k, v)
    for b, h in ((0, 0), (3, 17), (7, 31)):
        want = np_attention(q[b, h], k[b, h], v[b, h])
        assert np.allclose(got[b, h], want, rtol=1e-2, atol=1e-2), (b, h, np.abs(got[b, h] - want).max())


@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
def test_attention_fused_with_the_scale_behind_the_cast(dt):
    # the same graph with the scores scaled in fp32 (cast first, then the multiply): recognised as well
    rng = np.random.default_rng(77)
    conv = (lambda x: x.astype(np.float16)) if dt == "float16" else _bf16
    q, k, v = (conv(rng.standard_normal((3, n, 128))) for n in (200, 320, 320))
    t = Tester("mix")
    dts = dt if dt == "bfloat16" else None
    lq, lk, lv = t.load(q, dts), t.load(k, dts), t.load(v, dts)
    x = t.mul(t.cast(t.matmul(lq, lk, False, True), "float32"), 1.0 / math.sqrt(128))
    e = t.exp(t.sub(x, t.max(x, (2,), True)))
    out = t.store(t.matmul(t.cast(t.div(e, t.sum(e, (2,), True)), dt), lv, False, False))
    t.run()
    assert "entry attention" in t.das() and t.num_launches() == 1, t.das()
    got = t.output(out)
    got = Tester.convert_from_bf16(got) if dt == "bfloat16" else got
    want = np_attention(q, k, v)
    assert np.allclose(got, want, rtol=1e-2, atol=1e-2), np.abs(got - want).max()


@pytest.mark.parametrize("waves", ["8", "4"])
@pytest.mark.parametrize("shape", [((2, 3), 256, 192), ((1,), 64, 64), ((3,), 100, 128), ((2,), 300, 1024), ((), 513, 640)])
@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
def test_attention_fused_head_dimension_64(monkeypatch, shape, dt, waves):
    # the same kernel built for a head dimension of 64 (one 64-wide tile per K and V block instead of two)
    monkeypatch.setenv("DVM_ATTN_WAVES", waves)
    batch, sq, skv = shape
    rng = np.random.default_rng(sq + 1)
    conv = (lambda x: x.astype(np.float16)) if dt == "float16" else _bf16
    q, k, v = (conv(rng.standard_normal(batch + (n, 64))) for n in (sq, skv, skv))
    got = _fused(q, k, v, dt)
    want = np_attention(q, k, v)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-2, atol=1e-2), np.abs(got - want).max()


def test_attention_head_dimension_64_constant_values():
    # every row of V equal to c: the output rows are c whatever the scores; V = one-hot rows pick out softmax weights
    rng = np.random.default_rng(5)
    q, k = (rng.standard_normal((2, n, 64)).astype(np.float16) for n in (130, 192))
    v = np.tile(np.linspace(-1, 1, 64, dtype=np.float16), (2, 192, 1))
    got = _fused(q, k, v)
    assert np.allclose(got, v[:, :1, :].astype(np.float32), atol=2e-3), np.abs(got - v[:, :1, :]).max()
    v = np.zeros((2, 192, 64), np.float16)
    v[:, np.arange(64) * 3, np.arange(64)] = 1.0  # output column d = weight of key 3 d
    got = _fused(q, k, v).astype(np.float64)
    s = np.matmul(q.astype(np.float64), np.swapaxes(k.astype(np.float64), -1, -2)) / 8.0
    w = np.exp(s - s.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    assert np.allclose(got, w[:, :, ::3], rtol=1e-2, atol=1e-3), np.abs(got - w[:, :, ::3]).max()


@pytest.mark.parametrize("waves", ["8", "4"])
@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("sq,skv", [(100, 100), (197, 197), (64, 77), (300, 1), (33, 63), (256, 65), (40, 1000)])
def test_attention_fused_with_a_short_last_block_of_keys(monkeypatch, waves, d, sq, skv):
    # key counts that are no multiple of 64: the rows past the end are fetched from the last key and their scores masked.
    # Large values in V would show a weight that leaked through the mask.
    monkeypatch.setenv("DVM_ATTN_WAVES", waves)
    rng = np.random.default_rng(sq * 1000 + skv)
    q, k = (rng.standard_normal((2, n, d)).astype(np.float16) for n in (sq, skv))
    v = (rng.standard_normal((2, skv, d)) * 4).astype(np.float16)
    got = _fused(q, k, v)
    want = np_attention(q, k, v)
    assert np.allclose(got, want, rtol=1e-2, atol=2e-2), np.abs(got - want).max()


# ---- views as operands of the fused kernel: read in place, one launch ----

@pytest.mark.parametrize("b,s,h,d", [(2, 320, 4, 128), (1, 200, 3, 64), (2, 512, 2, 128)])
@pytest.mark.parametrize("how", ["view_load", "permute"])
def test_attention_on_sequence_major_tensors_read_heads_first(b, s, h, d, how):
    # q, k, v stored [batch, seq, heads, d] and read as [batch, heads, seq, d]; the result is dense, heads first
    rng = np.random.default_rng(b * 1000 + s + h)
    q, k, v = (rng.standard_normal((b, s, h, d)).astype(np.float16) for _ in range(3))
    t = Tester("mix")
    if how == "view_load":
        stride = [s * h * d, d, h * d, 1]
        lq, lk, lv = (t.view_load([b, h, s, d], stride, x) for x in (q, k, v))
    else:
        lq, lk, lv = (t.permute(t.load(x), [0, 2, 1, 3]) for x in (q, k, v))
    out = t.store(attention_graph(t, lq, lk, lv, 1.0 / math.sqrt(d), 4))
    t.run()
    assert "entry attention" in t.das() and "view, strides" in t.das() and t.num_launches() == 1, t.das()
    want = np_attention(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3))
    assert np.allclose(t.output(out), want, rtol=1e-2, atol=1e-2)


def test_attention_on_a_window_of_a_longer_key_value_cache():
    # k, v are the first skv rows of a cache [heads, 1024, d]; q dense (a dense operand beside views)
    rng = np.random.default_rng(77)
    hds, sq, skv, d, cap = 6, 128, 333, 128, 1024
    q = rng.standard_normal((hds, sq, d)).astype(np.float16)
    kc, vc = (rng.standard_normal((hds, cap, d)).astype(np.float16) for _ in range(2))
    t = Tester("mix")
    lk = t.slice_load(kc, [0, 0, 0], [hds, skv, d])
    lv = t.slice_load(vc, [0, 8, 0], [hds, skv, d])  # (a window that starts inside the cache)
    out = t.store(attention_graph(t, t.load(q), lk, lv, 1.0 / math.sqrt(d), 3))
    t.run()
    assert "entry attention" in t.das() and t.num_launches() == 1, t.das()
    assert np.allclose(t.output(out), np_attention(q, kc[:, :skv], vc[:, 8:8 + skv]), rtol=1e-2, atol=1e-2)


def test_attention_views_the_kernel_cannot_walk_run_unfused():
    # a head dimension that is not contiguous in memory: three launches, same result
    rng = np.random.default_rng(78)
    hds, s, d = 2, 128, 64
    q, v = (rng.standard_normal((hds, s, d)).astype(np.float16) for _ in range(2))
    kt = rng.standard_normal((hds, d, s)).astype(np.float16)  # K stored transposed
    t = Tester("mix")
    lk = t.view_load([hds, s, d], [d * s, 1, s], kt)
    out = t.store(attention_graph(t, t.load(q), lk, t.load(v), 1.0 / math.sqrt(d), 3))
    t.run()
    assert "entry attention" not in t.das(), t.das()
    assert np.allclose(t.output(out), np_attention(q, kt.transpose(0, 2, 1), v), rtol=1e-2, atol=1e-2)


# ---- the result written through strides: no dense copy of it exists ----

@pytest.mark.parametrize("b,s,h,d", [(2, 320, 4, 128), (1, 200, 3, 64), (2, 512, 2, 128)])
@pytest.mark.parametrize("how", ["permute_store", "view_store"])
@pytest.mark.parametrize("operands", ["dense", "views"])
def test_attention_result_written_sequence_major(b, s, h, d, how, operands):
    # the result [batch, heads, seq, d] goes to memory as [batch, seq, heads, d] (what the projection behind an
    # attention reads), as the dense Store of a Permute or as a Store with a stride list: one launch either way
    rng = np.random.default_rng(b * 1000 + s + h + 5)
    t = Tester("mix")
    if operands == "dense":
        q, k, v = (rng.standard_normal((b, h, s, d)).astype(np.float16) for _ in range(3))
        lq, lk, lv = (t.load(x) for x in (q, k, v))
        want = np_attention(q, k, v)
    else:
        q, k, v = (rng.standard_normal((b, s, h, d)).astype(np.float16) for _ in range(3))
        lq, lk, lv = (t.permute(t.load(x), [0, 2, 1, 3]) for x in (q, k, v))
        want = np_attention(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3))
    o = attention_graph(t, lq, lk, lv, 1.0 / math.sqrt(d), 4)
    if how == "permute_store":
        out = t.store(t.permute(o, [0, 2, 1, 3]))
        t.run()
        got = t.output(out)
    else:
        out = t.view_store(o, [s * h * d, d, h * d, 1], b * s * h * d)
        t.run()
        got = t.output(out, (b, s, h, d))
    assert "entry attention" in t.das() and "o: view, strides row=%d" % (h * d) in t.das() and t.num_launches() == 1, t.das()
    assert got.shape == (b, s, h, d) and np.allclose(got, want.transpose(0, 2, 1, 3), rtol=1e-2, atol=1e-2)


def test_attention_result_into_a_padded_buffer_and_results_the_kernel_cannot_place():
    rng = np.random.default_rng(91)
    hds, s, d = 3, 200, 128
    q, k, v = (rng.standard_normal((hds, s, d)).astype(np.float16) for _ in range(3))
    want = np_attention(q, k, v)
    # rows 160 elements apart, heads a whole number of rows apart: the kernel writes it in place
    t = Tester("mix")
    out = t.view_store(attention_graph(t, t.load(q), t.load(k), t.load(v), 1.0 / math.sqrt(d), 3), [s * 160, 160, 1], hds * s * 160)
    t.run()
    assert t.num_launches() == 1 and "o: view, strides row=160" in t.das(), t.das()
    got = t.output(out, (hds, s, 160))
    assert np.allclose(got[:, :, :d], want, rtol=1e-2, atol=1e-2) and not got[:, :, d:].any()
    # a transposing permute of the result (the head dimension no longer innermost) is a copy behind the kernel
    t = Tester("mix")
    out = t.store(t.permute(attention_graph(t, t.load(q), t.load(k), t.load(v), 1.0 / math.sqrt(d), 3), [0, 2, 1]))
    t.run()
    assert "entry attention" in t.das() and t.num_launches() == 2, t.das()
    assert np.allclose(t.output(out), want.transpose(0, 2, 1), rtol=1e-2, atol=1e-2)
    # a result with a second consumer keeps its dense copy
    t = Tester("mix")
    o = attention_graph(t, t.load(q), t.load(k), t.load(v), 1.0 / math.sqrt(d), 3)
    out1 = t.store(t.permute(o, [1, 0, 2]))
    out2 = t.store(t.mul(o, 2.0))
    t.run()
    assert np.allclose(t.output(out1), want.transpose(1, 0, 2), rtol=1e-2, atol=1e-2)
    assert np.allclose(t.output(out2), want * 2, rtol=1e-2, atol=2e-2)
