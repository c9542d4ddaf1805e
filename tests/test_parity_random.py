"""Parity on seeded random graphs (tests/random_graphs.py): the HIP path against the CPU oracle on graphs nobody
wrote by hand. Integer and bool outputs bit-exact, floating point 2e-4 (matmul 2e-2 on 16-bit operands)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from oracle.oracle import OracleKernel
from tests import random_graphs as R

gpu = pytest.mark.gpu
CHUNK = 100


def _read(t, st):
    out = t.output(st)
    if str(st.dtype()).endswith("bfloat16") or out.dtype == np.uint16:
        out = Tester.convert_from_bf16(out)
    return out


def _oracle(build):
    with np.errstate(all="ignore"):
        o = OracleKernel()
        return [o.output(s) for s in build(o)]


def _check(case, build, ker, refs, skip=()):
    t = Tester(ker)
    try:
        sts = build(t)
        t.run()
    except RuntimeError as e:
        if any(s in str(e) for s in skip):
            return
        raise AssertionError("case %d: %s" % (case, e))
    for i, (st, ref) in enumerate(zip(sts, refs)):
        assert R.close_enough(_read(t, st), ref, np.asarray(ref).dtype.kind in "ib"), "case %d output %d" % (case, i)


@gpu
@pytest.mark.parametrize("first,big,more", [(f, False, False) for f in range(0, 4 * CHUNK, CHUNK)] +
                         [(f, True, False) for f in range(0, 12 * CHUNK, CHUNK)] + [(f, True, True) for f in range(0, 12 * CHUNK, CHUNK)])
def test_pointwise_and_reduce_graphs(first, big, more):
    for case in range(first, first + CHUNK):
        build = R.pointwise_reduce_graph(case, big, more)
        try:
            refs = _oracle(build)
        except Exception:
            continue  # the plan produced a graph the oracle rejects
        _check(case, build, "", refs, skip=("not supported",))


@gpu
@pytest.mark.parametrize("first", range(0, 4 * CHUNK, CHUNK))
def test_typed_graphs(first):
    for case in range(first, first + CHUNK):
        build = R.typed_graph(case)
        _check(case, build, "", _oracle(build))


@gpu
@pytest.mark.parametrize("first", range(0, 2 * CHUNK, CHUNK))
def test_matmul_graphs(first):
    for case in range(first, first + CHUNK):
        build = R.matmul_graph(case)
        refs = _oracle(build)
        t = Tester("mix")
        sts = build(t)
        t.run()
        for i, (st, ref) in enumerate(zip(sts, refs)):
            out = _read(t, st).astype(np.float64)
            assert out.shape == ref.shape and np.allclose(out, ref.astype(np.float64), rtol=2e-2, atol=2e-2, equal_nan=True), \
                "case %d output %d %s" % (case, i, build.desc)


@gpu
@pytest.mark.parametrize("first", range(0, 4 * CHUNK, CHUNK))
def test_view_graphs(first):
    for case in range(first, first + CHUNK):
        build = R.view_graph(case)
        try:
            refs = _oracle(build)
        except Exception:
            continue  # the graph itself is invalid (an empty slice)
        _check(case, build, "", refs, skip=("needs a Copy", "not supported", "too many"))


@gpu
@pytest.mark.parametrize("first", range(0, 4 * CHUNK, CHUNK))
def test_one_dynamic_kernel_on_three_shapes(first):
    for case in range(first, first + CHUNK):
        with np.errstate(all="ignore"):
            insts, dts, tape, n_out, refs = R.dynamic_case(case)
        t = Tester(["vector:dyn", "split:dyn"][case % 2])
        loads = [t.load([-1], dt) for dt in dts]
        vals = [t.cast(l, "float32") for l in loads]
        for step in tape:
            vals.append(R.dyn_apply(t, vals, step))
        sts = [t.store(v) for v in vals[-n_out:]]
        for r, (ins, ref) in enumerate(zip(insts, refs)):
            for l, a in zip(loads, ins):
                t.input(l, a)
            t.run()
            for i, (st, want) in enumerate(zip(sts, ref)):
                assert R.close_enough(t.output(st), want, False), "case %d run %d output %d" % (case, r, i)


def test_random_graphs_compile_without_a_gpu():
    # the host side alone (emitter, partition, schedules) on a sample of the same graphs, in disassembly mode
    for case in range(60):
        for gen, ker in ((lambda c: R.pointwise_reduce_graph(c, True), ""), (R.typed_graph, ""), (R.matmul_graph, "mix"), (R.view_graph, "")):
            build = gen(case)
            try:
                _oracle(build) if gen is not R.matmul_graph else None
            except Exception:
                continue
            t = Tester(ker, run_mode="das")
            try:
                build(t)
                t.codegen()
            except RuntimeError as e:
                assert any(s in str(e) for s in ("needs a Copy", "not supported", "too many")), "case %d: %s" % (case, e)
                continue
            assert "== sub-kernel" in t.das() or t.das() == ""


@gpu
@pytest.mark.parametrize("first", range(0, 120, 30))
def test_attention_shapes(first):
    # examples/03_attention.py:20-50 at random sizes: head dim 128 takes the fused kernel (any number of queries and
    # keys, ragged tiles included), other head dims the three-launch path; 1e-2 against NumPy as in the example
    import math
    from tests.test_parity_attention import attention_graph, np_attention, _bf16
    for case in range(first, first + 30):
        rng = np.random.default_rng(7000 + case)
        batch = [(), (1,), (3,), (2, 2)][int(rng.integers(0, 4))]
        d = 128 if rng.random() < 0.7 else int(rng.choice([8, 64, 72, 256]))
        sq = int(rng.choice([1, 5, 31, 32, 33, 64, 100, 127, 129, 255, 256, 400, 700]))
        skv = int(rng.choice([1, 7, 63, 64, 65, 128, 200, 511, 513, 1000, 3000]))
        dt = "float16" if rng.random() < 0.5 else "bfloat16"
        conv = (lambda x: x.astype(np.float16)) if dt == "float16" else _bf16
        q, k, v = (conv(rng.standard_normal(batch + (n, d))) for n in (sq, skv, skv))
        t = Tester("mix")
        dts = dt if dt == "bfloat16" else None
        out = t.store(attention_graph(t, t.load(q, dts), t.load(k, dts), t.load(v, dts), 1.0 / math.sqrt(d), q.ndim, dt))
        t.run()
        got = _read(t, out)
        want = np_attention(q, k, v)
        assert got.shape == want.shape, (case, got.shape, want.shape)
        assert np.allclose(got, want, rtol=1e-2, atol=1e-2), (case, batch, sq, skv, d, dt, float(np.abs(got - want).max()))


@gpu
@pytest.mark.parametrize("first", range(0, 4 * CHUNK, CHUNK))
def test_index_graphs(first):
    for case in range(first, first + CHUNK):
        build = R.index_graph(case)
        _check(case, build, "", _oracle(build), skip=("needs a Copy",))
