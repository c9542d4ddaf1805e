"""Shared parity harness: one graph-building function runs on the HIP path
(dvm_amd.tester.Tester, through the C ABI) and on the CPU oracle
(oracle.oracle.OracleKernel); outputs are compared with each other and, when
given, with a NumPy golden."""
import numpy as np

from dvm_amd import DataType
from dvm_amd.tester import Tester, default_tolerance
from oracle.oracle import OracleKernel

# one tolerance policy for the harness and the parity tests
DEFAULT_EPS = {int(t): default_tolerance(t) for t in (DataType.float32, DataType.float16, DataType.bfloat16)}


def run_parity(build, arrays, dtypes=None, ker="vector", eps=None, golden=None, golden_eps=None, use_oracle=True):
    """build(k, *inputs) -> value or list of values. Returns the HIP outputs.

    use_oracle=False (sizes the scalar oracle cannot finish in seconds) checks against the golden only."""
    dtypes = dtypes or [None] * len(arrays)
    assert use_oracle or golden is not None
    t = Tester(ker)
    t_in = [t.load(a, d) for a, d in zip(arrays, dtypes)]
    t_out = build(t, *t_in)
    if not isinstance(t_out, (list, tuple)):
        t_out = [t_out]
    stores = [t.store(x) for x in t_out]
    if use_oracle:
        o = OracleKernel()
        o_out = build(o, *[o.load(a, d) for a, d in zip(arrays, dtypes)])
        if not isinstance(o_out, (list, tuple)):
            o_out = [o_out]
        refs = [o.output(o.store(x)) for x in o_out]
    else:
        refs = [None] * len(stores)
    t.run()
    outs = []
    for i, (s, ref) in enumerate(zip(stores, refs)):
        out = t.output(s)
        dt = int(s.dtype())
        if dt == int(DataType.bfloat16):
            out = Tester.convert_from_bf16(out)
        if ref is None:
            outs.append(out)
            continue
        assert out.shape == ref.shape, "output %d: shape %s vs oracle %s" % (i, out.shape, ref.shape)
        if dt in (int(DataType.int32), int(DataType.bool)):
            assert np.array_equal(out, ref), "output %d differs from the oracle (bit-exact required)\n%s" % (i, t.das())
        else:
            e = eps if eps is not None else DEFAULT_EPS[dt]
            assert np.allclose(out.astype(np.float32), ref.astype(np.float32), rtol=e, atol=e, equal_nan=True), (
                "output %d differs from the oracle beyond %g: max abs diff %g\n%s"
                % (i, e, np.nanmax(np.abs(out.astype(np.float64) - ref.astype(np.float64))), t.das()))
        outs.append(out)
    if golden is not None:
        g = golden if isinstance(golden, (list, tuple)) else [golden]
        for i, (out, gi) in enumerate(zip(outs, g)):
            if gi is None:
                continue
            dt = int(stores[i].dtype())
            e = golden_eps if golden_eps is not None else (eps if eps is not None else DEFAULT_EPS.get(dt, 0))
            assert np.allclose(out, gi, rtol=e, atol=e, equal_nan=True), (
                "output %d differs from the NumPy golden beyond %g\n%s" % (i, e, t.das()))
    return outs


def run_graph(ker, build, oracle=True, oracle_eps=None, min_launches=None):
    """build(k) builds a graph on k (the HIP Tester or the CPU oracle, same method names) and returns a list of
    (store, golden, eps) with golden a NumPy array / scalar or None. Checks the HIP outputs against the oracle's
    (usual tolerances, or oracle_eps) and against the goldens (eps, or the usual tolerance when None).
    Returns the Tester."""
    t = Tester(ker)
    specs = build(t)
    refs = None
    if oracle:
        o = OracleKernel()
        refs = [o.output(s[0]) for s in build(o)]
    t.run()
    if min_launches is not None:
        assert t.num_launches() >= min_launches, t.das()
    for i, (st, gold, eps) in enumerate(specs):
        out = t.output(st)
        dt = int(st.dtype())
        if dt == int(DataType.bfloat16):
            out = Tester.convert_from_bf16(out)
        exact = dt in (int(DataType.int32), int(DataType.bool))
        if refs is not None:
            ref = refs[i]
            assert out.shape == ref.shape, "output %d: shape %s vs oracle %s" % (i, out.shape, ref.shape)
            if exact:
                assert np.array_equal(out, ref), "output %d differs from the oracle (bit-exact required)\n%s" % (i, t.das())
            else:
                e = oracle_eps if oracle_eps is not None else DEFAULT_EPS[dt]
                assert np.allclose(out.astype(np.float32), ref.astype(np.float32), rtol=e, atol=e, equal_nan=True), (
                    "output %d differs from the oracle beyond %g\n%s" % (i, e, t.das()))
        if gold is not None:
            e = eps if eps is not None else DEFAULT_EPS.get(dt, 0)
            assert np.allclose(out, gold, rtol=e, atol=e, equal_nan=True), (
                "output %d differs from the NumPy golden beyond %g: max abs diff %g\n%s"
                % (i, e, np.nanmax(np.abs(np.asarray(out, np.float64) - np.asarray(gold, np.float64))), t.das()))
    return t
