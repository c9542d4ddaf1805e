"""GPU parity: matmul sub-kernels (MFMA tile loop + fused epilogue) against the CPU oracle and the
NumPy formulas of the reference's own tests (tests/ut/test_matmul.py, examples/04_matmul.py)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_parity

pytestmark = pytest.mark.gpu


def _mm(a, b, ta=False, tb=False):
    a, b = a.astype(np.float32), b.astype(np.float32)
    if ta:
        a = np.swapaxes(a, -1, -2)
    if tb:
        b = np.swapaxes(b, -1, -2)
    return np.matmul(a, b)


def _bf16(x):
    return Tester.convert_from_bf16(Tester.convert_to_bf16(x.astype(np.float32)))


def test_matmul_basic():  # tests/ut/test_matmul.py:17-41
    rng = np.random.default_rng(1)
    a, b = rng.random([128, 64]).astype(np.float16), rng.random([64, 32]).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, False, False), [a, b], ker="mix", golden=_mm(a, b).astype(np.float16))


@pytest.mark.parametrize("trans", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("size", [256, 1024])
def test_matmul_trans(trans, size):  # tests/ut/test_matmul.py:46-57
    rng = np.random.default_rng(size)
    a, b = rng.normal(0, 0.1, [size, size]).astype(np.float16), rng.normal(0, 0.1, [size, size]).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, *trans), [a, b], ker="mix", golden=_mm(a, b, *trans).astype(np.float16),
               use_oracle=size <= 256)


@pytest.mark.parametrize("trans", [(False, True), (True, True), (False, False), (True, False)])
@pytest.mark.parametrize("mnk", [(300, 5000, 4096), (1024, 4096, 8192), (4, 4096, 8192)])
def test_matmul_long_k(mnk, trans):  # tests/ut/test_matmul.py:62-77 (k cut to keep the CPU golden in seconds)
    m, n, k = mnk
    rng = np.random.default_rng(m)
    a = rng.normal(0, 0.1, [k, m] if trans[0] else [m, k]).astype(np.float16)
    b = rng.normal(0, 0.1, [n, k] if trans[1] else [k, n]).astype(np.float16)
    run_parity(lambda kk, x, y: kk.matmul(x, y, *trans), [a, b], ker="mix", golden=_mm(a, b, *trans).astype(np.float16), eps=2e-3,
               use_oracle=False)


def test_batchmatmul_unaligned_long_k():  # tests/ut/test_matmul.py:80-91
    rng = np.random.default_rng(3)
    a, b = rng.normal(0, 0.01, [2, 17, 65537]).astype(np.float16), rng.normal(0, 0.01, [65537, 19]).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, False, False), [a, b], ker="mix", golden=_mm(a, b).astype(np.float16), eps=2e-3)


@pytest.mark.parametrize("shapes", [
    ([2, 4, 256, 256], [2, 4, 256, 256]), ([256, 444], [3, 1, 444, 256]), ([1, 1, 256, 256], [3, 4, 256, 256]),
    ([3, 4, 256, 256], [1, 4, 256, 256]), ([3, 4, 256, 256], [256, 256]), ([1, 4, 256, 256], [3, 1, 256, 256]),
    ([4, 1, 10, 256], [256, 256]), ([24, 1, 4, 4], [4, 4096])])
def test_batchmatmul(shapes):  # tests/ut/test_matmul.py:96-116
    rng = np.random.default_rng(len(shapes[0]))
    a, b = rng.normal(0, 0.1, shapes[0]).astype(np.float16), rng.normal(0, 0.1, shapes[1]).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, False, False), [a, b], ker="mix", golden=_mm(a, b).astype(np.float16),
               use_oracle=False)


@pytest.mark.parametrize("shapes", [([4, 1, 256, 256], [1, 8, 256, 256]), ([768, 1024], [1024, 10240]), ([4, 10, 1, 256], [256, 256])])
def test_matmul_post_fusion(shapes):  # tests/ut/test_matmul.py:121-141
    rng = np.random.default_rng(5)
    a, b = rng.normal(0, 0.1, shapes[0]).astype(np.float16), rng.normal(0, 0.1, shapes[1]).astype(np.float16)
    c = _mm(a, b)
    z = rng.normal(0, 0.1, c.shape).astype(np.float32)
    t = Tester("mix")
    e = t.abs(t.add(t.cast(t.matmul(t.load(a), t.load(b), False, False), "float32"), t.load(z)))
    t.store_expect(e, np.abs(c + z), 2e-3)
    assert t.run_check()
    assert t.num_launches() == 1, t.das()  # the add and abs ride in the matmul's epilogue


def test_matmul_bf16():  # tests/ut/test_matmul.py:146-157
    rng = np.random.default_rng(6)
    a, b = _bf16(rng.normal(0, 0.1, [64, 64])), _bf16(rng.normal(0, 0.1, [64, 64]))
    run_parity(lambda k, x, y: k.matmul(x, y, False, False), [a, b], dtypes=["bfloat16", "bfloat16"], ker="mix",
               golden=_mm(a, b), eps=5e-3)


@pytest.mark.parametrize("shapes", [([211, 211], [211, 230]), ([193, 193], [193, 1930]), ([1, 1024], [1024, 320]), ([70000, 10], [10, 32])])
def test_unaligned_matmul(shapes):  # tests/ut/test_matmul.py:162-178
    rng = np.random.default_rng(7)
    a, b = rng.normal(0, 0.1, shapes[0]).astype(np.float16), rng.normal(0, 0.1, shapes[1]).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, False, False), [a, b], ker="mix", golden=_mm(a, b).astype(np.float16),
               use_oracle=shapes[0][0] < 1000)


@pytest.mark.parametrize("shapes", [([256, 256], [256, 256]), ([32, 256], [256, 128]), ([2048, 1024], [1024, 5120])])
@pytest.mark.parametrize("row", [True, False])
def test_matmul_post_broadcast_fusion(shapes, row):  # tests/ut/test_matmul.py:183-228
    rng = np.random.default_rng(8)
    a, b = rng.normal(0, 0.1, shapes[0]).astype(np.float16), rng.normal(0, 0.1, shapes[1]).astype(np.float16)
    c = _mm(a, b)
    z = rng.normal(0, 0.1, [c.shape[1]] if row else [c.shape[0], 1]).astype(np.float32)
    run_parity(lambda k, x, y, zz: k.abs(k.add(k.cast(k.matmul(x, y, False, False), "float32"), zz)), [a, b, z], ker="mix",
               golden=np.abs(c + z), eps=2e-3, use_oracle=shapes[0][0] <= 256)


@pytest.mark.parametrize("shapes", [([211, 211], [211, 230]), ([193, 100], [100, 257]), ([1, 127], [127, 127]), ([1, 1000], [1000, 4000]),
                                    ([123, 1], [1, 777])])
def test_unaligned_matmul_post_fusion(shapes):  # tests/ut/test_matmul.py:233-252
    rng = np.random.default_rng(9)
    a, b = rng.normal(0, 0.1, shapes[0]).astype(np.float16), rng.normal(0, 0.1, shapes[1]).astype(np.float16)
    run_parity(lambda k, x, y: k.add(k.cast(k.matmul(x, y, False, False), "float32"), 2.5), [a, b], ker="mix",
               golden=_mm(a, b) + 2.5, eps=2e-3)


def test_matmul_post_fusion_two_outputs():  # tests/ut/test_matmul.py:257-302
    rng = np.random.default_rng(10)
    a, b = rng.normal(0, 0.1, [1024, 512]).astype(np.float16), rng.normal(0, 0.1, [512, 1024]).astype(np.float16)
    c = _mm(a, b).astype(np.float16)
    z = rng.normal(0, 0.1, c.shape).astype(np.float16)

    def build(k, zz, x, y):
        zh = k.mul(zz, 0.5)
        cc = k.matmul(x, y, False, False)
        d = k.sub(k.add(k.add(cc, zh), 0.1), zh)
        return [cc, d]
    run_parity(build, [z, a, b], ker="mix", golden=[c, c + np.float16(0.1)], eps=2e-3, use_oracle=False)


@pytest.mark.parametrize("batch", [(), ((1, 2), (3, 1))])
def test_matmul_transposed_b_odd_sizes(batch):  # tests/ut/test_matmul.py:307-345
    rng = np.random.default_rng(11)
    sa, sb = ([800, 1024], [700, 1024]) if not batch else ([1, 2, 800, 1024], [3, 1, 700, 1024])
    a, b = rng.normal(0, 0.1, sa).astype(np.float16), rng.normal(0, 0.1, sb).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, False, True), [a, b], ker="mix", golden=_mm(a, b, False, True).astype(np.float16),
               use_oracle=False)


def test_long_epilogue():  # tests/ut/test_matmul.py:350-373 (smaller m and n)
    rng = np.random.default_rng(12)
    a, b = rng.normal(0, 0.1, [1024, 1152]).astype(np.float16), rng.normal(0, 0.1, [1152, 512]).astype(np.float16)
    c, d = rng.normal(0, 0.1, [1024, 512]).astype(np.float16), rng.normal(0, 0.1, [512]).astype(np.float32)
    mm = _mm(a, b)

    def build(k, aa, bb, cc, dd):
        y1 = k.cast(k.matmul(aa, bb, False, False), "float32")
        y3 = k.add(k.cast(cc, "float32"), dd)
        y6 = k.mul(y1, k.mul(y3, k.mul(y3, y3)))
        for _ in range(100):
            y6 = k.add(y6, 0.1)
        return [y3, k.cast(y6, "float16")]
    run_parity(build, [a, b, c, d], ker="mix", golden=[c + d, (c.astype(np.float32) + d) ** 3 * mm + 10], eps=2e-3, use_oracle=False)


@pytest.mark.parametrize("shapes", [([2, 16, 128, 128], [1, 128, 256]), ([16, 16], [16, 4096]), ([1344, 1792], [1792, 64]),
                                    ([1024, 1024], [1024, 4096])])
@pytest.mark.parametrize("dt", ["float16", "bfloat16"])
def test_matmul_bias(shapes, dt):  # tests/ut/test_matmul.py:398-435
    rng = np.random.default_rng(13)
    conv = (lambda x: x.astype(np.float16)) if dt == "float16" else _bf16
    a, b = conv(rng.normal(0, 0.1, shapes[0])), conv(rng.normal(0, 0.1, shapes[1]))
    c = _mm(a, b)
    z = conv(rng.normal(0, 0.1, [c.shape[-1]]))
    dts = [None] * 3 if dt == "float16" else ["bfloat16"] * 3
    run_parity(lambda k, x, y, zz: k.matmul(x, y, False, False, zz), [a, b, z], dtypes=dts, ker="mix",
               golden=c + z.astype(np.float32), eps=2e-3 if dt == "float16" else 1e-2, use_oracle=shapes[0][0] <= 64)


@pytest.mark.parametrize("shapes", [([16, 16], [16, 4096]), ([4096, 16], [16, 16]), ([32, 4096, 16], [16, 16]), ([512, 64], [64, 8192])])
def test_matmul_short_k(shapes):  # tests/ut/test_matmul.py:440-455
    rng = np.random.default_rng(14)
    a, b = rng.normal(0, 0.1, shapes[0]).astype(np.float16), rng.normal(0, 0.1, shapes[1]).astype(np.float16)
    run_parity(lambda k, x, y: k.matmul(x, y, False, False), [a, b], ker="mix", golden=_mm(a, b), eps=2e-3, use_oracle=False)


def test_dyn_matmul():  # tests/ut/test_matmul.py:482-509 (one kernel object, new shapes every call)
    t = Tester("mix:dyn")
    x, y, z = t.load([-1, -1], "float16"), t.load([-1, -1], "float16"), t.load([-1, -1], "float16")
    out = t.store(t.add(t.matmul(x, y, False, False), z))
    rng = np.random.default_rng(15)
    for xs, ys, zs in [([256, 128], [128, 256], [256, 256]), ([1000, 4096], [4096, 256], [1000, 1]), ([256, 128], [128, 512], [256, 1]),
                       ([444, 3333], [3333, 1111], [1, 1111]), ([1024, 1024], [1024, 2222], [1024, 2222]), ([2560, 128], [128, 512], [512])]:
        xd, yd, zd = (rng.normal(0, 0.1, s).astype(np.float16) for s in (xs, ys, zs))
        t.input(x, xd)
        t.input(y, yd)
        t.input(z, zd)
        t.run()
        assert t.check(out, _mm(xd, yd).astype(np.float16) + zd, 2e-3)


@pytest.mark.parametrize("case", [([2000, 512], [512, 3000], [1, 3000]), ([2000, 512], [512, 3000], [2000, 1]), ([2048, 512], [512, 4096], [1, 1]),
                                  ([3, 4, 256, 512], [3, 4, 512, 512], [1, 4, 256, 512]), ([3, 4, 256, 512], [3, 4, 512, 512], [3, 1, 256, 512]),
                                  ([3, 4, 256, 512], [3, 4, 512, 512], [256, 512]), ([3, 4, 256, 512], [512, 512], [1, 1, 256, 512]),
                                  ([3, 4, 256, 512], [3, 4, 512, 512], [3, 1, 1, 512]), ([3, 4, 256, 512], [3, 4, 512, 512], [3, 1, 256, 1]),
                                  ([3, 4, 256, 512], [3, 4, 512, 512], [1])])
def test_post_fusion_broadcast(case):  # tests/ut/test_matmul.py:514-545
    rng = np.random.default_rng(16)
    a, b = rng.normal(0, 0.1, case[0]).astype(np.float16), rng.normal(0, 0.1, case[1]).astype(np.float16)
    z = rng.normal(0, 0.1, case[2]).astype(np.float16)
    run_parity(lambda k, x, y, zz: k.add(k.matmul(x, y, False, False), zz), [a, b, z], ker="mix",
               golden=_mm(a, b).astype(np.float16) + z, eps=2e-3, use_oracle=False)


def test_matmul_bias_silu_cast_example():  # examples/04_matmul.py (BASELINE config 5 at a size the oracle finishes)
    rng = np.random.default_rng(17)
    m, n, k = 256, 192, 128
    a, b, bias = _bf16(rng.normal(0, 0.1, [m, k])), _bf16(rng.normal(0, 0.1, [k, n])), rng.normal(0, 0.1, [n]).astype(np.float32)

    def build(kk, x, y, bb):
        h = kk.add(kk.cast(kk.matmul(x, y, False, False), "float32"), bb)
        s = kk.div(h, kk.add(kk.exp(kk.mul(h, -1.0)), 1.0))
        return kk.cast(s, "bfloat16")
    h = _bf16(_mm(a, b)) + bias
    t = run_parity(build, [a, b, bias], dtypes=["bfloat16", "bfloat16", None], ker="mix", golden=_bf16(h / (1 + np.exp(-h))), eps=1e-2)
    assert t[0].shape == (m, n)
