"""GPU parity: products whose k axis is shared between workgroups (two launches: fp32 partial tiles, then their sum
and the epilogue). The reference's split-k cases (tests/ut/test_matmul.py:60-76, eps 2e-3) with the split the host
chooses by itself, and forced splits over every tile size, layout and the guarded path (ragged tiles, k not a
multiple of 64), with an epilogue, with batches, and twice in a row for bit-equal results (no atomics: the partials
are added in a fixed order)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def _operands(rng, m, n, k, ta, tb, dtype, sigma=0.1, batch=()):
    af = (rng.standard_normal(list(batch) + ([k, m] if ta else [m, k])) * sigma).astype(np.float32)
    bf = (rng.standard_normal(list(batch) + ([n, k] if tb else [k, n])) * sigma).astype(np.float32)
    if dtype == "bfloat16":
        a16, b16 = Tester.convert_to_bf16(af), Tester.convert_to_bf16(bf)
        return a16, b16, Tester.convert_from_bf16(a16), Tester.convert_from_bf16(b16)
    a16, b16 = af.astype(np.float16), bf.astype(np.float16)
    return a16, b16, a16.astype(np.float32), b16.astype(np.float32)


def _load(t, x16, dtype):
    if dtype == "bfloat16":
        x = t.load(x16.shape, "bfloat16")
        t.input(x, x16)
        return x
    return t.load(x16)


def _product(a_ref, b_ref, ta, tb):
    return np.matmul(np.swapaxes(a_ref, -1, -2) if ta else a_ref, np.swapaxes(b_ref, -1, -2) if tb else b_ref)


@pytest.mark.parametrize("m,n,k", [[300, 5000, 40000], [1024, 4096, 32768], [4, 4096, 32768]])
@pytest.mark.parametrize("trans", [[False, True], [True, True], [False, False], [True, False]])
def test_matmul_split_k(m, n, k, trans):  # tests/ut/test_matmul.py:60-76
    rng = np.random.default_rng(m + 7 * int(trans[0]) + 3 * int(trans[1]))
    a16, b16, a_ref, b_ref = _operands(rng, m, n, k, trans[0], trans[1], "float16")
    expect = _product(a_ref, b_ref, trans[0], trans[1]).astype(np.float16)
    t = Tester("mix")
    c = t.matmul(t.load(a16), t.load(b16), trans[0], trans[1])
    t.store_expect(c, expect, 2e-3)
    assert t.run_check()


def test_the_host_splits_a_long_k_axis_of_a_product_with_few_tiles():
    # 16 tiles of 256x256 (or 64 of 128x128) for 256 compute units and k = 16384: split; a product that fills the chip: not
    rng = np.random.default_rng(5)
    for (m, n, k), want in [((1024, 1024, 16384), True), ((4096, 4096, 1024), False), ((256, 256, 64), False)]:
        a16, b16, a_ref, b_ref = _operands(rng, m, n, k, False, False, "bfloat16")
        t = Tester("mix")
        out = t.store(t.matmul(_load(t, a16, "bfloat16"), _load(t, b16, "bfloat16"), False, False))
        t.run()
        das = t.das()
        assert ("split-k partials" in das) == want, das
        assert ("split-k sum of" in das) == want, das
        assert t.num_launches() == (2 if want else 1)
        got = Tester.convert_from_bf16(t.output(out)).astype(np.float64)
        ref = _product(a_ref.astype(np.float64), b_ref.astype(np.float64), False, False)
        assert np.allclose(got, ref, rtol=1e-2, atol=1e-2), float(np.abs(got - ref).max())


@pytest.mark.parametrize("tile", ["256", "128", "64"])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_forced_split_on_every_tile_and_layout(monkeypatch, tile, dtype, ta, tb):
    # full tiles plus a ragged tile in m and n (guarded path), three parts of unequal length (k = 1216: 448 + 448 + 320),
    # a bias row that must be added once, not once per part, and a second operand in the epilogue
    monkeypatch.setenv("DVM_CUBE_TILE", tile)
    monkeypatch.setenv("DVM_CUBE_SPLITK", "3")
    m, n, k = 512 + 40, 512 + 24, 1216
    rng = np.random.default_rng(int(tile) + 2 * int(ta) + int(tb))
    a16, b16, a_ref, b_ref = _operands(rng, m, n, k, ta, tb, dtype, sigma=0.125)
    bias = rng.standard_normal([n]).astype(np.float32)
    other = rng.standard_normal([m, n]).astype(np.float32)
    t = Tester("mix")
    c = t.cast(t.matmul(_load(t, a16, dtype), _load(t, b16, dtype), ta, tb), "float32")
    out = t.store(t.mul(t.add(c, t.load(bias)), t.load(other)))
    t.run()
    das = t.das()
    assert "split-k partials 3 x 448" in das and "split-k sum of 3" in das and ("tile=" + tile) in das, das
    prod = _product(a_ref.astype(np.float64), b_ref.astype(np.float64), ta, tb)
    want = (prod + bias) * other
    got = t.output(out).astype(np.float64)
    # the product is rounded to the operand type before the bias joins it: half a unit in its last place, scaled by `other`
    bound = 1e-2 + 1e-2 * np.abs(want) + 2.0 ** (-8 if dtype == "bfloat16" else -11) * np.abs(prod * other)
    assert (np.abs(got - want) <= bound).all(), float((np.abs(got - want) - bound).max())


@pytest.mark.parametrize("k", [1000, 130, 4096 + 8])
def test_forced_split_with_a_k_axis_that_is_no_multiple_of_64(monkeypatch, k):
    monkeypatch.setenv("DVM_CUBE_SPLITK", "4")
    rng = np.random.default_rng(k)
    m, n = 192, 320
    a16, b16, a_ref, b_ref = _operands(rng, m, n, k, False, True, "float16")
    t = Tester("mix")
    out = t.store(t.matmul(t.load(a16), t.load(b16), False, True))
    t.run()
    assert "split-k partials" in t.das() and "guarded" in t.das(), t.das()
    want = _product(a_ref.astype(np.float64), b_ref.astype(np.float64), False, True)
    got = t.output(out).astype(np.float64)
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3), float(np.abs(got - want).max())


def test_split_product_with_batches_and_silu(monkeypatch):
    # [3, 2, m, k] x [2, k, n] (the outer batch axis of B is broadcast), bias + SiLU, bf16 store
    monkeypatch.setenv("DVM_CUBE_SPLITK", "2")
    rng = np.random.default_rng(21)
    m, n, k = 256, 384, 2048
    af = (rng.standard_normal([3, 2, m, k]) / 32).astype(np.float32)
    bf = (rng.standard_normal([2, k, n])).astype(np.float32)
    a16, b16 = Tester.convert_to_bf16(af), Tester.convert_to_bf16(bf)
    bias = (rng.standard_normal([n]) * 0.1).astype(np.float32)
    t = Tester("mix")
    z = t.cast(t.matmul(_load(t, a16, "bfloat16"), _load(t, b16, "bfloat16"), False, False, t.load(bias)), "float32")
    y = t.div(z, t.add(t.exp(t.mul(z, -1.0)), 1.0))
    out = t.store(t.cast(y, "bfloat16"))
    t.run()
    assert "split-k partials 2 x 1024" in t.das(), t.das()
    zr = np.matmul(Tester.convert_from_bf16(a16).astype(np.float64), Tester.convert_from_bf16(b16).astype(np.float64)) + bias
    want = zr / (1.0 + np.exp(-zr))
    got = Tester.convert_from_bf16(t.output(out)).astype(np.float64)
    assert np.allclose(got, want, rtol=1e-2, atol=1e-2), float(np.abs(got - want).max())


def test_split_results_are_the_same_bits_on_every_run(monkeypatch):
    monkeypatch.setenv("DVM_CUBE_SPLITK", "8")
    rng = np.random.default_rng(33)
    a16, b16, _, _ = _operands(rng, 512, 512, 8192, False, False, "float16", sigma=1.0)
    outs = []
    for _ in range(3):
        t = Tester("mix")
        out = t.store(t.cast(t.matmul(t.load(a16), t.load(b16), False, False), "float32"))
        t.run()
        assert "split-k sum of 8" in t.das()
        outs.append(t.output(out).copy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_split_against_the_unsplit_product(monkeypatch):
    # fp32 partial sums in a different association: the 16-bit results agree except where the fp32 sums straddle a
    # rounding boundary (one unit in the last place there)
    rng = np.random.default_rng(34)
    a16, b16, _, _ = _operands(rng, 384, 640, 4096, False, True, "float16", sigma=0.25)
    res = {}
    for split in ["0", "4"]:
        monkeypatch.setenv("DVM_CUBE_SPLITK", split)
        t = Tester("mix")
        out = t.store(t.matmul(t.load(a16), t.load(b16), False, True))
        t.run()
        assert ("split-k" in t.das()) == (split != "0")
        res[split] = t.output(out).astype(np.float32)
    differ = res["0"] != res["4"]
    assert differ.mean() < 0.02, float(differ.mean())
    assert np.allclose(res["0"], res["4"], rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("tile", ["256", "128", "64"])
@pytest.mark.parametrize("parts", [5, 7, 13])
def test_part_counts_that_leave_the_last_group_of_partials_short(monkeypatch, tile, parts):
    # the second launch reads the partial tiles in groups of four (tile 256, 64) or eight (tile 128): 5, 7 and 13 parts
    # leave a last group of one, three, five or seven; the result must be the sum of exactly `parts` partials
    monkeypatch.setenv("DVM_CUBE_TILE", tile)
    monkeypatch.setenv("DVM_CUBE_SPLITK", str(parts))
    m, n, k = 256 + 8, 320, parts * 128
    rng = np.random.default_rng(parts * 1000 + int(tile))
    a16, b16, a_ref, b_ref = _operands(rng, m, n, k, False, True, "float16", sigma=0.25)
    t = Tester("mix")
    out = t.store(t.cast(t.matmul(t.load(a16), t.load(b16), False, True), "float32"))
    t.run()
    assert ("split-k sum of %d" % parts) in t.das(), t.das()
    want = _product(a_ref.astype(np.float64), b_ref.astype(np.float64), False, True)
    got = t.output(out).astype(np.float64)
    # fp32 accumulation, the product rounded to fp16 before the cast back
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3), float(np.abs(got - want).max())
