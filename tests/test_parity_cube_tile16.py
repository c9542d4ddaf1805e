"""GPU parity of the matmul epilogue's one-pass route (VCF_DUMP16): every product's program starts with [add of a bias
row] [rounding to the operand type] (the matmul's value, src/vm_aic.cce:34-470), and the kernel does these two where
the accumulators are, keeps the rounded tile in local memory as 16-bit values and walks the rest of the program over
the whole tile in one pass. With DVM_CUBE_DUMP16=0 the tile goes through local memory as fp32, half a tile per pass,
and the interpreter does the two instructions itself: the same arithmetic in the same order, so both routes must
give the same bits. Each case is also checked against np.matmul on fp32 copies (tests/ut/test_matmul.py:34-36).
Shapes cover all three tile sizes, edge tiles, batches, a bias of each float type and a split k axis."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def _operand(rng, shape, dtype, scale=0.25):
    x = rng.standard_normal(shape, dtype=np.float32) * scale
    return Tester.convert_to_bf16(x) if dtype == "bfloat16" else x.astype(dtype)


def _f32(x, dtype):
    return Tester.convert_from_bf16(x) if dtype == "bfloat16" else x.astype(np.float32)


EPILOGUES = {
    "plain": lambda t, z: z,
    "relu": lambda t, z: t.maximum(z, 0.0),
    "silu": lambda t, z: t.div(z, t.add(t.exp(t.mul(z, -1.0)), 1.0)),
    "affine_abs": lambda t, z: t.abs(t.add(t.mul(z, 0.5), 1.0)),
    "floor": lambda t, z: t.floor(t.mul(z, 4.0)),  # (not one of the slim pass's operators: the full interpreter)
}


def _run(monkeypatch, on, dtype, m, n, k, bias_dtype, epi, batch=()):
    monkeypatch.setenv("DVM_CUBE_DUMP16", "1" if on else "0")
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = _operand(rng, list(batch) + [m, k], dtype)
    b = _operand(rng, list(batch) + [k, n], dtype)
    bias = None if bias_dtype is None else _operand(rng, [n], bias_dtype, 1.0)
    t = Tester("mix")
    la, lb = t.load(a.shape, dtype), t.load(b.shape, dtype)
    t.input(la, a)
    t.input(lb, b)
    if bias is None:
        mm = t.matmul(la, lb, False, False)
    else:
        lbias = t.load(bias.shape, bias_dtype)
        t.input(lbias, bias)
        mm = t.matmul(la, lb, False, False, lbias)
    z = t.cast(mm, "float32")
    out = t.store(t.cast(EPILOGUES[epi](t, z), dtype) if epi != "plain" else mm)
    t.run()
    return t.output(out), t.das(), (a, b, bias)


@pytest.mark.parametrize("epi", sorted(EPILOGUES))
@pytest.mark.parametrize("dtype,bias_dtype", [("bfloat16", "float32"), ("float16", "float16"), ("bfloat16", None), ("float16", "float32"),
                                              ("bfloat16", "bfloat16")])
@pytest.mark.parametrize("m,n,k", [(512, 512, 128), (300, 264, 96), (1024, 2048, 64), (100, 72, 40), (2048, 1024, 256)])
def test_one_pass_route_gives_the_bits_of_the_two_pass_route(monkeypatch, epi, dtype, bias_dtype, m, n, k):
    got, das_on, (a, b, bias) = _run(monkeypatch, True, dtype, m, n, k, bias_dtype, epi)
    ref, das_off, _ = _run(monkeypatch, False, dtype, m, n, k, bias_dtype, epi)
    assert "tile-as-16-bit" in das_on and "tile-as-16-bit" not in das_off, das_on
    assert np.array_equal(got, ref), das_on
    if epi in ("plain", "relu"):
        z = np.matmul(_f32(a, dtype), _f32(b, dtype)) + (0.0 if bias is None else _f32(bias, bias_dtype))
        want = np.maximum(z, 0.0) if epi == "relu" else z
        assert np.allclose(_f32(got, dtype), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("batch,m,n,k", [((3,), 200, 136, 64), ((2, 2), 256, 256, 128)])
def test_batches(monkeypatch, batch, m, n, k):
    got, das_on, (a, b, bias) = _run(monkeypatch, True, "float16", m, n, k, "float32", "silu", batch)
    ref, _, _ = _run(monkeypatch, False, "float16", m, n, k, "float32", "silu", batch)
    assert "tile-as-16-bit" in das_on, das_on
    assert np.array_equal(got, ref), das_on
    z = (np.matmul(a.astype(np.float32), b.astype(np.float32)) + bias.astype(np.float32)).astype(np.float16).astype(np.float32)
    assert np.allclose(got.astype(np.float32), z / (1.0 + np.exp(-z)), rtol=2e-2, atol=2e-2)


def test_split_k_sum_goes_the_one_pass_route_too(monkeypatch):
    # 1024 x 1024 x 16384: sixteen 256-tiles, the k axis shared between workgroups; the launch that adds the partial
    # tiles runs the same epilogue
    got, das_on, (a, b, bias) = _run(monkeypatch, True, "bfloat16", 1024, 1024, 16384, "float32", "relu")
    ref, _, _ = _run(monkeypatch, False, "bfloat16", 1024, 1024, 16384, "float32", "relu")
    assert "split-k sum" in das_on and "tile-as-16-bit" in das_on, das_on
    assert np.array_equal(got, ref), das_on


@pytest.mark.parametrize("act", ["silu", "sigmoid", "silu_as_product"])
@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
@pytest.mark.parametrize("shape", [(512, 384, 128), (300, 520, 64), (2048, 1024, 256)])
def test_fused_activation_instructions_give_the_bits_of_the_separate_ones(monkeypatch, act, dt, shape):
    # x / (exp(-x) + 1) and 1 / (exp(-x) + 1) behind a matmul are one epilogue instruction each (VU_SILU_APPROX,
    # VU_SIGMOID_APPROX): the same fp32 operations in the same order as the three or four they replace
    m, n, k = shape
    rng = np.random.default_rng(m + n + k)
    a = (rng.standard_normal([m, k]) * 0.3).astype(np.float32)
    b = (rng.standard_normal([k, n]) * 0.3).astype(np.float32)
    bias = rng.standard_normal([n]).astype(np.float32)

    def run():
        t = Tester("mix")
        la, lb = (t.load(v.astype(np.float16)) if dt == "float16" else t.load(v, dt) for v in (a, b))
        h = t.add(t.cast(t.matmul(la, lb, False, False), "float32"), t.load(bias))
        if act == "silu":
            y = t.div(h, t.add(t.exp(t.mul(h, -1.0)), 1.0))
        elif act == "sigmoid":
            y = t.div(1.0, t.add(t.exp(t.mul(h, -1.0)), 1.0))
        else:
            y = t.mul(h, t.div(1.0, t.add(t.exp(t.mul(h, -1.0)), 1.0)))
        out = t.store(t.cast(y, dt))
        t.run()
        return t.output(out), t.das()

    fused, das = run()
    assert ("SiLU~" in das) == (act == "silu") and ("Sigmoid~" in das) == (act != "silu"), das
    monkeypatch.setenv("DVM_CUBE_FUSE_ACT", "0")
    apart, das0 = run()
    assert "SiLU~" not in das0 and "Sigmoid~" not in das0 and "RDiv~" in das0, das0
    assert np.array_equal(fused.view(np.uint16), apart.view(np.uint16))
    # and against float64
    h64 = a.astype(np.float64) @ b.astype(np.float64)
    ref = None
    if dt == "float16":
        h64 = (a.astype(np.float16).astype(np.float64) @ b.astype(np.float16).astype(np.float64)).astype(np.float16).astype(np.float64) + bias
        ref = h64 / (np.exp(-h64) + 1) if act != "sigmoid" else 1 / (np.exp(-h64) + 1)
        assert np.allclose(fused.astype(np.float64), ref, rtol=3e-3, atol=3e-3)
