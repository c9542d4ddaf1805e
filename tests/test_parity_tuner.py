"""GPU: the online tuner of matmul launches (Config::SetOnlineTuner / SetLazyTuner, include/dvm.h:735-738 of the
reference; its table of tuned tile parameters, src/ops_m.h:174-263). With the tuner on, the first code generation of a
product shape times every (block tile, parts of the k axis) candidate on the device and remembers the fastest; the
result does not depend on the choice beyond the order of the fp32 additions along k, so tuned and untuned runs agree to
the matmul tolerance of the reference's tests (tests/ut/test_matmul.py:34-36), and the measured choice is no slower
than the host's own rule."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def _product(m, k, n, batch=(), trans_b=False, epilogue=False, seed=0):
    rng = np.random.default_rng(seed)
    a = (rng.standard_normal(list(batch) + [m, k], dtype=np.float32) * 0.25).astype(np.float16)
    b = (rng.standard_normal(list(batch) + ([n, k] if trans_b else [k, n]), dtype=np.float32) * 0.25).astype(np.float16)
    t = Tester("mix")
    c = t.matmul(t.load(a), t.load(b), False, trans_b)
    if epilogue:
        c = t.cast(t.maximum(t.cast(c, "float32"), 0.0), "float16")
    out = t.store(c)
    t.run()
    got = t.output(out).astype(np.float32)
    want = np.matmul(a.astype(np.float32), np.swapaxes(b, -1, -2).astype(np.float32) if trans_b else b.astype(np.float32))
    if epilogue:
        want = np.maximum(want.astype(np.float16).astype(np.float32), 0.0)
    assert np.allclose(got, want, rtol=2e-2, atol=2e-2)
    return t


@pytest.fixture
def tuner():
    Tester.tuner_clear()
    Tester.set_online_tuning(True)
    yield
    Tester.set_online_tuning(False)
    Tester.set_lazy_tuning(False)
    Tester.tuner_clear()


SHAPES = [(512, 4096, 512), (1024, 1024, 1024), (200, 8192, 136), (4096, 256, 4096), (64, 16384, 64)]


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_tuned_choice_is_measured_once_and_is_no_slower(tuner, m, k, n):
    measured0, _ = Tester.tuner_stats()
    t = _product(m, k, n)
    measured1, size1 = Tester.tuner_stats()
    assert measured1 == measured0 + 1 and size1 >= 1
    tuned = sorted(t.perf_samples(warmup=2, iters=8))[4]
    das_tuned = t.das()
    # the same shape again: the table answers, nothing is measured, the same program comes out
    t2 = _product(m, k, n, seed=1)
    assert Tester.tuner_stats()[0] == measured1 and t2.das().splitlines()[1].split(" blocks=")[0] == das_tuned.splitlines()[1].split(" blocks=")[0]
    # with an epilogue behind the product the shape's entry is used as well
    _product(m, k, n, epilogue=True)
    assert Tester.tuner_stats()[0] == measured1
    Tester.set_online_tuning(False)
    t3 = _product(m, k, n)
    plain = sorted(t3.perf_samples(warmup=2, iters=8))[4]
    assert tuned <= plain * 1.15 + 2.0, (tuned, plain, das_tuned, t3.das())


def test_batches_transposes_and_the_lazy_switch(tuner):
    Tester.set_online_tuning(False)
    Tester.set_lazy_tuning(True)   # either switch tunes at the first code generation of a shape
    _product(192, 512, 320, batch=(6,), trans_b=True)
    assert Tester.tuner_stats()[0] >= 1
    n0 = Tester.tuner_stats()[1]
    _product(192, 512, 320, batch=(6,), trans_b=False)   # another layout is another entry
    assert Tester.tuner_stats()[1] == n0 + 1


def test_without_a_tuner_nothing_is_measured():
    Tester.tuner_clear()
    before = Tester.tuner_stats()
    _product(256, 256, 256)
    assert Tester.tuner_stats() == before
