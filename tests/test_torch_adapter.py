"""GPU: `@kernel` functions called with torch tensors (the custom fused operator route of the reference's
docs/pytorch.md): inputs are read in place, outputs are torch tensors, launches go to torch's current stream.

The checks run in a process of their own that imports torch first: torch brings its own copy of the HIP runtime,
and a process in which the device layer of this package has already loaded the system's copy cannot initialise
torch's afterwards (torch then reports that it finds no device). In the other order both share torch's copy."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

_SCRIPT = r'''
import numpy as np
import torch
import dvm_amd as dvm


@dvm.kernel(ktype="split", dynamic=True)
def add_rms(k, x, r, w):
    h = k.cast(k.add(k.load(x, dvm.bfloat16), k.load(r, dvm.bfloat16)), dvm.float32)
    ss = k.sum(k.mul(h, h), (1,), True)
    rstd = k.div(1.0, k.sqrt(k.add(k.mul(ss, 1.0 / 512), 1e-6)))
    return k.store(k.cast(k.mul(k.mul(h, rstd), k.load(w, dvm.float32)), dvm.bfloat16))


g = torch.Generator(device="cuda").manual_seed(7)
w = torch.rand(512, device="cuda", generator=g) * 0.2 + 0.9
for rows in (33, 257, 33):  # shapes change between calls, nothing is copied to the host
    x = torch.randn(rows, 512, device="cuda", generator=g).to(torch.bfloat16)
    r = torch.randn(rows, 512, device="cuda", generator=g).to(torch.bfloat16)
    out = add_rms(x, r, w)
    assert isinstance(out, torch.Tensor) and out.is_cuda and out.dtype == torch.bfloat16 and tuple(out.shape) == (rows, 512)
    h = (x + r).float()  # the bf16 sum rounded once, as the kernel's Add.bf16
    want = h * torch.rsqrt((h * h).mean(1, keepdim=True) + 1e-6) * w
    torch.cuda.synchronize()
    assert torch.allclose(out.float(), want, rtol=1e-2, atol=1e-2)
print("tensors in place: ok")


@dvm.kernel(ktype="vector", dynamic=True)
def scale(k, x):
    return k.store(k.mul(k.load(x, dvm.float32), 3.0))


side = torch.cuda.Stream()
x = torch.zeros(1 << 22, device="cuda")
with torch.cuda.stream(side):
    x.fill_(2.0)           # queued on the side stream, the kernel after it on the same stream
    y = scale(x)
    z = y + 1.0            # and torch's own consumer after the kernel
side.synchronize()
assert float(z.min()) == 7.0 and float(z.max()) == 7.0
print("current stream: ok")

try:
    scale(torch.zeros(8, device="cuda", dtype=torch.float16))
    raise SystemExit("a tensor of the wrong type was accepted")
except TypeError:
    pass
assert np.allclose(scale(np.ones(8, np.float32)), 3.0)  # the numpy route still works on the same kernel
print("type check: ok")

# ---- outputs supplied by the caller (docs/pytorch.md:238-239 of the reference: run(..., out_buffer)) ----
x = torch.randn(1000, 300, device="cuda", generator=g)
buf = torch.full((1000, 300), -1.0, device="cuda")
ret = scale(x, out=buf)
torch.cuda.synchronize()
assert ret is buf and torch.equal(buf, x * 3.0)
for bad in (torch.empty(300, 1000, device="cuda"), torch.empty(1000, 300, device="cuda", dtype=torch.float16),
            torch.empty(1000, 600, device="cuda")[:, ::2]):
    try:
        scale(x, out=bad)
        raise SystemExit("an output tensor of the wrong shape, type or layout was accepted")
    except TypeError:
        pass
print("caller's outputs: ok")


# ---- tensors that are not contiguous are read through their strides, not copied ----
@dvm.kernel(ktype="split", dynamic=True)
def row_norm(k, x):
    v = k.load(x, dvm.float32)
    m = k.mul(k.sum(v, (1,), True), 1.0 / 256)
    return k.store(k.sub(v, m))


base = torch.randn(512, 1024, device="cuda", generator=g)
window = base[100:400, 256:512]                # rows of 256 elements, 1024 apart
out = row_norm(window)
assert "view" in row_norm.das() or "k[1024]" in row_norm.das(), row_norm.das()  # the load walks the window in place
torch.cuda.synchronize()
assert torch.allclose(out, window - window.mean(1, keepdim=True), rtol=1e-5, atol=1e-5)
tr = torch.randn(256, 300, device="cuda", generator=g).t()   # a transposed tensor: element-by-element reads, still in place
out = row_norm(tr)
torch.cuda.synchronize()
assert torch.allclose(out, tr - tr.mean(1, keepdim=True), rtol=1e-5, atol=1e-5)
out = row_norm(base[:300, :256].contiguous())  # and a dense tensor on the same kernel object afterwards
torch.cuda.synchronize()
assert torch.allclose(out, base[:300, :256] - base[:300, :256].mean(1, keepdim=True), rtol=1e-5, atol=1e-5)


@dvm.kernel(ktype="mix", dynamic=True)
def proj(k, a, w):
    return k.store(k.matmul(k.load(a, dvm.float16), k.load(w, dvm.float16), False, False))


a = (torch.randn(256, 512, device="cuda", generator=g) / 8).half()
wide = (torch.randn(512, 1024, device="cuda", generator=g) / 8).half()
out = proj(a, wide[:, 128:640])                # a window of a wider weight: the matmul walks it through its leading dimension
torch.cuda.synchronize()
assert torch.allclose(out.float(), a.float() @ wide[:, 128:640].float(), rtol=2e-2, atol=2e-2)
print("strided tensors: ok")


# ---- the workspace of a kernel with several launches comes from torch's allocator ----
@dvm.kernel(ktype="split", dynamic=True)
def col_softmax(k, x):
    v = k.load(x, dvm.float32)
    e = k.exp(k.sub(v, k.max(v, (0,), True)))
    return k.store(k.div(e, k.sum(e, (0,), True)))


xs = torch.randn(32000, 512, device="cuda", generator=g)
torch.cuda.synchronize()
before = torch.cuda.memory_allocated()
ys = col_softmax(xs)  # (new names: rebinding an earlier tensor would free it and blur the count)
assert col_softmax.num_launches() > 1 and col_softmax.workspace_bytes() > 0
assert torch.cuda.memory_allocated() >= before + ys.numel() * 4 + col_softmax.workspace_bytes()  # output + workspace, both torch's
torch.cuda.synchronize()
assert torch.allclose(ys, torch.softmax(xs, 0), rtol=1e-4, atol=1e-6)
print("workspace from torch: ok")
'''


def test_kernel_on_torch_tensors():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, "-c", _SCRIPT], cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stdout + r.stderr
    for line in ("tensors in place: ok", "current stream: ok", "type check: ok", "caller's outputs: ok", "strided tensors: ok",
                 "workspace from torch: ok"):
        assert line in r.stdout, r.stdout + r.stderr
