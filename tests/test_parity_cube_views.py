"""GPU parity: strided views as matmul operands. A view whose innermost or second-innermost stride is 1 is read
by the MFMA tile loop in place, through a leading dimension, batch strides and a base offset taken from the view
(the reference routes views into its cube unit as well: include/dvm.h:434-479, src/isa.h:1187-1452): a sliced weight
matrix, the heads-first view of a [batch, seq, heads, dim] tensor, a permuted batch, a transposed operand. Each
graph takes the same number of launches as its dense counterpart, runs on the CPU oracle as well and is checked
against np.matmul on fp32 copies (the golden of tests/ut/test_matmul.py:34-36)."""
import numpy as np
import pytest

from dvm_amd.tester import Tester
from tests.util import run_graph

pytestmark = pytest.mark.gpu


def row_major(shape):
    st = [1] * len(shape)
    for i in range(len(shape) - 1, 0, -1):
        st[i - 1] = st[i] * shape[i]
    return st


def f16(rng, shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float16)


def gold(a, b):
    return np.matmul(a.astype(np.float32), b.astype(np.float32))


@pytest.mark.parametrize("m,k,n,r0,c0", [(128, 256, 192, 64, 32), (300, 512, 264, 8, 8), (256, 256, 256, 5, 3), (64, 64, 64, 0, 8)])
def test_sliced_weight_matrix(m, k, n, r0, c0):
    # B is a [k, n] window of a larger weight: rows r0.., columns c0.. (an offset that is no multiple of 8 elements
    # takes the guarded staging path, the others the vector path)
    rng = np.random.default_rng(m + k + n)
    a = f16(rng, [m, k], 0.25)
    w = f16(rng, [k + r0 + 7, n + c0 + 24], 0.25)

    def build(t):
        lb = t.slice_load(w, [r0, c0], [k, n])
        return [(t.store(t.matmul(t.load(a), lb, False, False)), gold(a, w[r0:r0 + k, c0:c0 + n]), 2e-2)]

    t = run_graph("mix", build)
    assert t.num_launches() == 1, t.das()


@pytest.mark.parametrize("b,s,h,d", [(2, 256, 4, 64), (1, 300, 3, 128), (3, 128, 2, 32)])
def test_heads_first_view_of_a_sequence_major_tensor(b, s, h, d):
    # q, k of shape [b, s, h, d] read as [b, h, s, d]: scores = q k^T per head, without a copy of either
    rng = np.random.default_rng(b * 100 + s + h + d)
    q, k = f16(rng, [b, s, h, d], 0.3), f16(rng, [b, s, h, d], 0.3)
    stride = [s * h * d, d, h * d, 1]

    def build(t):
        lq = t.view_load([b, h, s, d], stride, q)
        lk = t.view_load([b, h, s, d], stride, k)
        return [(t.store(t.matmul(lq, lk, False, True)), gold(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 3, 1)), 2e-2)]

    t = run_graph("mix", build)
    assert t.num_launches() == 1, t.das()


def test_permute_of_a_loaded_value_as_operand():
    # the Permute operator on a load: [b, s, h, d] -> [b, h, s, d] as A, and a transposing permute as B
    rng = np.random.default_rng(3)
    b, s, h, d, n = 2, 192, 2, 64, 128
    x = f16(rng, [b, s, h, d], 0.3)
    w = f16(rng, [n, d], 0.3)  # stored [n, d]; the graph permutes it to [d, n]

    def build(t):
        lx = t.permute(t.load(x), [0, 2, 1, 3])
        lw = t.permute(t.load(w), [1, 0])
        return [(t.store(t.matmul(lx, lw, False, False)), gold(x.transpose(0, 2, 1, 3), w.T), 2e-2)]

    t = run_graph("mix", build)
    assert t.num_launches() == 1, t.das()


def test_permuted_batch_and_transposed_view():
    # A: a batch [b0, b1, m, k] stored as [b1, b0, m, k]; B: stored [b0, b1, n, k] and read as its transpose through
    # a stride list (the second-innermost stride is 1: the operand's transpose flag flips)
    rng = np.random.default_rng(4)
    b0, b1, m, k, n = 2, 3, 96, 128, 80
    a = f16(rng, [b1, b0, m, k], 0.3)
    bt = f16(rng, [b0, b1, n, k], 0.3)

    def build(t):
        la = t.view_load([b0, b1, m, k], [m * k, b0 * m * k, k, 1], a)
        lb = t.view_load([b0, b1, k, n], [b1 * n * k, n * k, 1, k], bt)
        return [(t.store(t.matmul(la, lb, False, False)), gold(a.transpose(1, 0, 2, 3), bt.transpose(0, 1, 3, 2)), 2e-2)]

    t = run_graph("mix", build)
    assert t.num_launches() == 1, t.das()


def test_view_operand_with_an_epilogue_and_big_tiles():
    # a 4096 x 4096 x 256 product on the 256 tile whose B operand is a window of a wider matrix, with a bias row behind it
    rng = np.random.default_rng(5)
    m, k, n = 4096, 256, 4096
    a = f16(rng, [m, k], 0.125)
    w = f16(rng, [k, n + 512], 0.125)
    bias = rng.standard_normal([n]).astype(np.float32)

    def build(t):
        lb = t.view_load([k, n], [n + 512, 1], w, offset=256)
        y = t.add(t.cast(t.matmul(t.load(a), lb, False, False), "float32"), t.load(bias))
        want = gold(a, w[:, 256:256 + n]).astype(np.float16).astype(np.float32) + bias
        return [(t.store(y), want, 2e-2)]

    t = run_graph("mix", build, oracle=False)  # (the scalar oracle would take a quarter of a minute; np.matmul is the golden)
    assert t.num_launches() == 1 and "tile=256" in t.das(), t.das()


def test_operand_without_a_contiguous_axis_is_refused():
    rng = np.random.default_rng(6)
    a = f16(rng, [64, 128])
    w = f16(rng, [128, 256])
    t = Tester("mix")
    lb = t.view_load([64, 64], [512, 2], w)  # every second column of every second row
    t.store(t.matmul(t.load(a[:, :64].copy()), lb, False, False))
    with pytest.raises(RuntimeError, match="no contiguous axis"):
        t.run()
