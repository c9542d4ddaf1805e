"""GPU parity: the graphs of the reference's pass tests (tests/ut/test_pass_dead_code_eliminate.py,
test_pass_eliminate_reshape.py) with the passes selected by name the way those tests do (`set_passes`). The pipeline
here is fixed: what DeadCodeEliminate achieves always happens (operators nothing stores are not compiled), a reshape
is a view (of a load: read in place; of a computed value: read from where it was written), the scheduling passes of
the reference's tile machine have no counterpart and are accepted by name. Results against NumPy, the effect against the listing."""
import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu


def test_dead_load_and_dead_operator_are_not_compiled():
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal([1000], dtype=np.float32), rng.standard_normal([1000], dtype=np.float32)
    t = Tester("split")
    x0 = t.load(a)
    t.load(b)            # nothing reads it
    t.sqrt(x0)           # nothing stores it
    t.store_expect(t.mul(x0, 0.6), a * np.float32(0.6))
    t.set_passes("DeadCodeEliminate")
    assert t.run_check()
    das = t.das()
    assert "Sqrt" not in das and das.count("load.fp32") == 1 and t.num_launches() == 1, das


@pytest.mark.parametrize("passes", [("EliminateReshape",), ("ReorderLoad", "ReorderStore", "CompactPeakLiveness"), ()])
def test_reshape_between_operators(passes):
    # (here a reshape of a computed value that changes the innermost axes is a launch boundary: the value is written
    # once, dense, and read through its new shape; whichever passes are named, the result is the same)
    rng = np.random.default_rng(1)
    a = rng.standard_normal([50, 256], dtype=np.float32)
    t = Tester("split")
    x = t.mul(t.reshape(t.add(t.load(a), 0.2), [25, 256, 2]), 0.3)
    t.store_expect(x, ((a + np.float32(0.2)).reshape([25, 256, 2]) * np.float32(0.3)))
    t.set_passes(*passes)
    assert t.run_check()
    assert t.num_launches() <= 2, t.das()


def test_reshape_of_a_load_is_a_copy_in_one_launch():
    rng = np.random.default_rng(2)
    a = rng.standard_normal([50, 256], dtype=np.float32)
    t = Tester("split")
    t.store_expect(t.reshape(t.load(a), [25, 256, 2]), a.reshape([25, 256, 2]))
    t.set_passes("EliminateReshape")
    assert t.run_check()
    assert t.num_launches() == 1, t.das()


def test_reshapes_behind_copies_of_a_transposing_view():
    # tests/ut/test_pass_eliminate_reshape.py:49-66 in a smaller shape: the view is copied (a launch that gathers),
    # the two reshapes behind the copies read that dense copy through their new shapes
    rng = np.random.default_rng(3)
    phys = rng.standard_normal([4, 6, 20, 64], dtype=np.float32)
    t = Tester("split")
    x = t.view_load([6, 20, 4, 64], [20 * 64, 64, 6 * 20 * 64, 1], phys)
    x = t.reshape(t.reshape(t.copy(t.copy(x)), [6, 20, 256]), [120, 256])
    t.store_expect(x, np.transpose(phys, (1, 2, 0, 3)).copy().reshape([120, 256]))
    t.set_passes("EliminateReshape")
    assert t.run_check()


def test_unknown_pass_name_is_refused():
    t = Tester("split")
    with pytest.raises(RuntimeError, match="unknown pass"):
        t.set_passes("UnrollEverything")
