"""GPU test of dvm_hip_launch_vm_static_ws (include/dvm_hip.h): the launch entry point that allocates nothing and
keeps the values one launch hands to the next in the library's own static workspace.

The kernel is an attention graph at head dimension 96, which the fused kernel does not take: three launches
(matmul, softmax with two chained reduces, matmul) and two values in the workspace. It runs through the existing
route first (dvm_rt_run: dvm_hip_launch_vm per launch, workspace from hipMalloc), then its exported programs go
through the new entry point via the C ABI of libdvm_hip.so; both results must agree bit for bit. Twice in a row on
one kernel object, the second time with a smaller input, so that what the first call left in the workspace is still
there when the second one starts."""
import ctypes
import math
import os

import numpy as np
import pytest

from dvm_amd.tester import Tester

pytestmark = pytest.mark.gpu

HIP_SO = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "dvm_amd", "lib", "libdvm_hip.so")
STATIC_WS_BYTES = 32 * 1024 * 1024
ERR_WS_TOO_LARGE, ERR_BAD_WS_WORD = -2, -3


def _hip():
    lib = ctypes.CDLL(HIP_SO)
    lib.dvm_hip_launch_vm_static_ws.restype = ctypes.c_int
    lib.dvm_hip_launch_vm_static_ws.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32),
                                                ctypes.POINTER(ctypes.c_uint32), ctypes.c_uint32, ctypes.c_size_t, ctypes.c_void_p]
    lib.dvm_hip_memset.restype = ctypes.c_int
    lib.dvm_hip_memset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
    lib.dvm_hip_synchronize_stream.restype = ctypes.c_int
    lib.dvm_hip_synchronize_stream.argtypes = [ctypes.c_void_p]
    lib.dvm_hip_error_string.restype = ctypes.c_char_p
    lib.dvm_hip_error_string.argtypes = [ctypes.c_int]
    return lib


def _pack(programs):
    """(blobs, geometry, ws word pairs, count of pairs) in the form the entry point takes."""
    blobs = b"".join(p[0] for p in programs)
    geo = (ctypes.c_uint32 * (3 * len(programs)))(*[v for p in programs for v in p[1]])
    pairs = [v for i, p in enumerate(programs) for w in p[2] for v in (i, w)]
    words = (ctypes.c_uint32 * max(1, len(pairs)))(*pairs)
    return ctypes.create_string_buffer(blobs, len(blobs)), geo, words, len(pairs) // 2


def _np_attention(q, k, v):
    s = np.matmul(q.astype(np.float32), np.swapaxes(k.astype(np.float32), -1, -2)) / math.sqrt(q.shape[-1])
    p = np.exp(s - s.max(-1, keepdims=True))
    return np.matmul(p / p.sum(-1, keepdims=True), v.astype(np.float32))


def test_static_workspace_launch_matches_the_allocating_route():
    hip = _hip()
    rng = np.random.default_rng(7)
    t = Tester("mix:dyn")
    lq, lk, lv = (t.load([1, 1, 96], "float16") for _ in range(3))  # (a head dimension the fused kernel does not take)
    s = t.mul(t.matmul(lq, lk, False, True), 1.0 / math.sqrt(96))
    x = t.cast(s, "float32")
    x = t.sub(x, t.max(x, (2,), True))
    e = t.exp(x)
    p = t.cast(t.div(e, t.sum(e, (2,), True)), "float16")
    out = t.store(t.matmul(p, lv, False, False))

    for heads, sq, skv in ((6, 384, 512), (2, 100, 192)):  # the second call is smaller than the first
        q, k, v = (rng.standard_normal((heads, n, 96)).astype(np.float16) for n in (sq, skv, skv))
        for load, arr in ((lq, q), (lk, k), (lv, v)):
            t.input(load, arr)
        t.run()  # the existing route
        want = t.output(out).copy()
        assert t.num_launches() == 3 and t.workspace_bytes() > 0, t.das()
        assert np.allclose(want, _np_attention(q, k, v), rtol=1e-2, atol=1e-2)

        programs = t.programs()
        assert sum(len(pr[2]) for pr in programs) >= 2  # values cross launches through the workspace
        blobs, geo, words, n_ws = _pack(programs)
        dst = t.device_ptr(out)
        assert hip.dvm_hip_memset(dst, 0, want.nbytes) == 0  # what the first route wrote is gone
        rc = hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, words, n_ws, t.workspace_bytes(), None)
        assert rc == 0, hip.dvm_hip_error_string(rc)
        assert hip.dvm_hip_synchronize_stream(None) == 0
        got = t.output(out)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), "heads=%d sq=%d skv=%d" % (heads, sq, skv)

    # sizes beyond the static workspace and malformed workspace words are refused before anything is launched
    rc = hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, words, n_ws, STATIC_WS_BYTES + 1, None)
    assert rc == ERR_WS_TOO_LARGE and b"DVM_HIP_STATIC_WS_BYTES" in hip.dvm_hip_error_string(rc)
    bad = (ctypes.c_uint32 * 2)(len(programs), 0)
    assert hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, bad, 1, t.workspace_bytes(), None) == ERR_BAD_WS_WORD
    assert hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, words, n_ws, 16, None) == ERR_BAD_WS_WORD  # offsets past ws_bytes


def test_static_workspace_holds_the_partials_of_shared_reduces_and_split_products():
    # two launches each, the first leaves fp32 partial results in the workspace: column sums of a [60000, 96] tensor
    # (a reduce shared between workgroups) and a 256x256x8192 product with its k axis split
    hip = _hip()
    rng = np.random.default_rng(8)
    x = rng.standard_normal([60000, 96]).astype(np.float32)
    a = (rng.standard_normal([256, 8192]) / 16).astype(np.float16)
    b = (rng.standard_normal([8192, 256]) / 16).astype(np.float16)
    kernels = []
    t = Tester("split")
    kernels.append((t, t.store(t.sum(t.load(x), (0,), True)), "shared-reduce parts="))
    t = Tester("mix")
    kernels.append((t, t.store(t.matmul(t.load(a), t.load(b), False, False)), "split-k partials"))
    for t, out, marker in kernels:
        t.run()
        want = t.output(out).copy()
        assert marker in t.das() and t.num_launches() == 2 and 0 < t.workspace_bytes() <= STATIC_WS_BYTES, t.das()
        programs = t.programs()
        blobs, geo, words, n_ws = _pack(programs)
        assert n_ws >= 2  # the partials are written by the first launch and read by the second
        assert hip.dvm_hip_memset(t.device_ptr(out), 0, want.nbytes) == 0
        rc = hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, words, n_ws, t.workspace_bytes(), None)
        assert rc == 0, hip.dvm_hip_error_string(rc)
        assert hip.dvm_hip_synchronize_stream(None) == 0
        assert np.array_equal(t.output(out).view(np.uint8), want.view(np.uint8)), marker


def test_static_workspace_passes_over_launches_with_nothing_to_do_and_refuses_a_word_listed_twice():
    # A kernel with a sub-kernel over an empty tensor: its exported program has the geometry {0, 0, 0}. The entry point
    # passes over it, as the allocating route does; the other programs still run, and every program is checked
    # against its geometry before the first one is launched.
    hip = _hip()
    rng = np.random.default_rng(9)
    x = rng.standard_normal([70000, 64]).astype(np.float32)
    t = Tester("split")
    out = t.store(t.sum(t.load(x), (0,), True))          # a shared reduce: two launches and a workspace
    t.store(t.mul(t.load(np.zeros([0, 16], np.float32)), 2.0))  # nothing to do
    t.run()
    want = t.output(out).copy()
    programs = t.programs()
    assert any(tuple(p[1]) == (0, 0, 0) for p in programs) and sum(1 for p in programs if tuple(p[1]) != (0, 0, 0)) == 2, [p[1] for p in programs]
    blobs, geo, words, n_ws = _pack(programs)
    assert hip.dvm_hip_memset(t.device_ptr(out), 0, want.nbytes) == 0
    rc = hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, words, n_ws, t.workspace_bytes(), None)
    assert rc == 0, hip.dvm_hip_error_string(rc)
    assert hip.dvm_hip_synchronize_stream(None) == 0
    assert np.array_equal(t.output(out).view(np.uint8), want.view(np.uint8))
    # the same workspace word listed twice would get the workspace address added twice: refused, nothing launched
    pairs = [v for i, p in enumerate(programs) for w in p[2] for v in (i, w)]
    twice = (ctypes.c_uint32 * (len(pairs) + 2))(*(pairs + pairs[:2]))
    assert hip.dvm_hip_memset(t.device_ptr(out), 0, want.nbytes) == 0
    assert hip.dvm_hip_launch_vm_static_ws(blobs, len(programs), geo, twice, n_ws + 1, t.workspace_bytes(), None) == ERR_BAD_WS_WORD
    assert hip.dvm_hip_synchronize_stream(None) == 0
    assert not t.output(out).any()
