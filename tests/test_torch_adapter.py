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
'''


def test_kernel_on_torch_tensors():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, "-c", _SCRIPT], cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stdout + r.stderr
    for line in ("tensors in place: ok", "current stream: ok", "type check: ok"):
        assert line in r.stdout, r.stdout + r.stderr
