"""Writes tests/golden/vectors.npz: small seeded inputs and their expected outputs for every operator family of
the hot path, computed with the NumPy formulas the reference's own tests use as goldens (file:line per case).
Nothing of the reference is imported or run. Re-run with `python tests/golden/make_golden.py` to regenerate."""
import math
import os

import numpy as np


def bf16_round(x):  # python/dvm/tester.py:93-99 (round to nearest even on the upper 16 bits)
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    return r.view(np.float32)


def main():
    rng = np.random.default_rng(20260101)
    v = {}
    # pointwise fp32 (tests/ut/test_elemwise.py:23-200)
    a = rng.normal(0, 2, [7, 33]).astype(np.float32)
    b = rng.normal(0, 2, [7, 33]).astype(np.float32)
    v["ew_a"], v["ew_b"] = a, b
    v["ew_add"], v["ew_sub"], v["ew_mul"], v["ew_div"] = a + b, a - b, a * b, a / b
    v["ew_max"], v["ew_min"] = np.maximum(a, b), np.minimum(a, b)
    v["ew_abs"], v["ew_exp"], v["ew_sqrt"], v["ew_log"] = np.abs(a), np.exp(a), np.sqrt(np.abs(a)), np.log(np.abs(a) + 1)
    v["ew_round"], v["ew_floor"], v["ew_ceil"], v["ew_trunc"] = np.round(a), np.floor(a), np.ceil(a), np.trunc(a)
    v["ew_gt"], v["ew_eq"] = a > b, a == a
    v["ew_select"] = np.where(a > b, a, b)
    # int32 wraps (src/vm_gpu.cu:262-266)
    ia = np.array([[np.iinfo(np.int32).min, -7, 0, 5, np.iinfo(np.int32).max]], np.int32)
    ib = np.array([[1, 3, -2, 5, 1]], np.int32)
    v["i_a"], v["i_b"] = ia, ib
    with np.errstate(over="ignore"):
        v["i_add"], v["i_mul"], v["i_abs"] = ia + ib, ia * ib, np.abs(ia)
    # fp16 / bf16: computed in fp32, rounded once (tests/ut/test_cast.py:25-51)
    h = rng.normal(0, 1, [5, 19]).astype(np.float16)
    v["h_a"] = h
    v["h_mul"] = (h.astype(np.float32) * h.astype(np.float32)).astype(np.float16)
    f = rng.normal(0, 3, [5, 19]).astype(np.float32)
    v["c_f32"], v["c_to_bf16"], v["c_to_f16"], v["c_to_i32"] = f, bf16_round(f), f.astype(np.float16), f.astype(np.int32)
    # broadcast and reduce (tests/ut/test_broadcast.py:24-165, tests/ut/test_reduce.py:24-115)
    r = rng.normal(-0.5, 0.5, [3, 10, 6, 7]).astype(np.float32)
    v["r_x"] = r
    v["r_sum_last"] = r.sum(3, keepdims=True, dtype=np.float64).astype(np.float32)
    v["r_sum_023"] = r.sum((0, 2, 3), keepdims=True, dtype=np.float64).astype(np.float32)
    v["r_max_1"], v["r_min_13"] = r.max(1), r.min((1, 3))
    v["b_row"] = rng.normal(0, 1, [1, 10, 1, 7]).astype(np.float32)
    v["b_add"] = r + v["b_row"]
    # batch-norm forward, training statistics (examples/02_batchnorm.py:19-24 with eps)
    x = rng.standard_normal([4, 6, 5, 5]).astype(np.float32)
    g, be = rng.uniform(0.5, 1.5, [1, 6, 1, 1]).astype(np.float32), rng.normal(0, 0.1, [1, 6, 1, 1]).astype(np.float32)
    x64 = x.astype(np.float64)
    v["bn_x"], v["bn_g"], v["bn_b"] = x, g, be
    v["bn_y"] = ((x64 - x64.mean((0, 2, 3), keepdims=True)) / np.sqrt(x64.var((0, 2, 3), keepdims=True) + 1e-5) * g + be).astype(np.float32)
    # matmul (tests/ut/test_matmul.py:34-36) and matmul + bias + SiLU (examples/04_matmul_post_fusion.py:53-58)
    ma, mb = rng.normal(0, 0.1, [48, 40]).astype(np.float16), rng.normal(0, 0.1, [40, 24]).astype(np.float16)
    v["mm_a"], v["mm_b"] = ma, mb
    v["mm_c"] = np.matmul(ma.astype(np.float32), mb.astype(np.float32)).astype(np.float16)
    bias = rng.normal(0, 0.1, [24]).astype(np.float32)
    z = v["mm_c"].astype(np.float32) + bias
    v["mm_bias"], v["mm_silu"] = bias, (z / (1 + np.exp(-z))).astype(np.float16)
    # attention (examples/03_attention.py:20-28)
    q, k, vv = (rng.normal(0, 0.5, s).astype(np.float16) for s in ((4, 8), (6, 8), (6, 12)))
    sc = np.matmul(q.astype(np.float32), k.astype(np.float32).T) / math.sqrt(8)
    pr = np.exp(sc - sc.max(-1, keepdims=True))
    v["at_q"], v["at_k"], v["at_v"] = q, k, vv
    v["at_o"] = np.matmul(pr / pr.sum(-1, keepdims=True), vv.astype(np.float32)).astype(np.float16)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz"), **v)


if __name__ == "__main__":
    main()
