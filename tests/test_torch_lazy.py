"""GPU: eager fusion without graphs (`dvm_amd.lazy_fusion`, the role of the reference's docs/pytorch.md section 4):
torch operators issued inside the block are captured into DVM graphs and run as fused launches; results are compared
with the same program run by torch alone. Runs in a process of its own that imports torch first (see
tests/test_torch_adapter.py for why)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

_SCRIPT = r'''
import torch
import torch.nn.functional as F
import dvm_amd as dvm

g = torch.Generator(device="cuda").manual_seed(11)
def rnd(*shape, dtype=torch.float32):
    return torch.randn(*shape, device="cuda", generator=g).to(dtype)

# ---- the reference's example (docs/pytorch.md section 4.1): one fused launch, the temporaries are never stored ----
x, y = rnd(1024, 1024), rnd(1024, 1024)
want = torch.sqrt(torch.abs(x) + torch.abs(y) + 1.0) * 0.5
with dvm.lazy_fusion() as lf:
    out = torch.sqrt(torch.abs(x) + torch.abs(y) + 1.0) * 0.5
torch.cuda.synchronize()
assert lf.stats["captured"] == 6 and lf.stats["flushes"] == 1 and lf.stats["launches"] == 1 and lf.stats["stored"] == 1, lf.stats
assert type(out) is torch.Tensor and torch.allclose(out, want, rtol=1e-6, atol=1e-6)
print("example: ok", lf.stats)

# ---- activations, compares, where, casts in three types ----
def acts(t):
    a = F.silu(t) + torch.sigmoid(t) * torch.tanh(t)
    b = F.gelu(t, approximate="tanh") - F.relu(t) + F.leaky_relu(t, 0.1)
    c = torch.where(t > 0.5, a, b * 2.0)
    d = torch.maximum(c, -t) / (torch.abs(t) + 1.0) - (1.5 - t)
    return d, (t <= 0.0)
for dt, tol in ((torch.float32, 1e-5), (torch.float16, 4e-3), (torch.bfloat16, 3e-2)):
    t = rnd(300, 257, dtype=dt)
    want_d, want_m = acts(t)
    with dvm.lazy_fusion() as lf:
        got_d, got_m = acts(t)
    torch.cuda.synchronize()
    assert got_d.dtype == dt and got_m.dtype == torch.bool and torch.equal(got_m, want_m)
    assert torch.allclose(got_d.float(), want_d.float(), rtol=tol, atol=tol), (dt, (got_d.float() - want_d.float()).abs().max())
    assert lf.stats["launches"] == 1 and lf.stats["stored"] == 2, lf.stats
print("activations: ok")

# ---- a normalisation with a reduce and a cast: one launch ----
h, w = rnd(333, 1024, dtype=torch.bfloat16), rnd(1024) * 0.1 + 1.0
def rms(h, w):
    hf = h.float()
    return (hf * torch.rsqrt((hf * hf).sum(-1, keepdim=True) / 1024 + 1e-6) * w).to(torch.bfloat16)
want = rms(h, w)
with dvm.lazy_fusion() as lf:
    got = rms(h, w)
torch.cuda.synchronize()
assert lf.stats["launches"] == 1 and lf.stats["fallbacks"] == 0, lf.stats
assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2)
print("rmsnorm: ok", lf.stats)

# ---- a linear layer with its activation: matmul, bias and SiLU in one launch; the weight is read transposed in place ----
a, wt, bias = rnd(512, 256, dtype=torch.bfloat16) * 0.1, rnd(384, 256, dtype=torch.bfloat16) * 0.1, rnd(384, dtype=torch.bfloat16)
want = F.silu(torch.addmm(bias, a, wt.t()))
with dvm.lazy_fusion() as lf:
    got = F.silu(torch.addmm(bias, a, wt.t()))
torch.cuda.synchronize()
assert lf.stats["launches"] == 1 and lf.stats["captured"] == 2, lf.stats
assert torch.allclose(got.float(), want.float(), rtol=3e-2, atol=3e-2)
lin = torch.nn.Linear(256, 384, device="cuda", dtype=torch.bfloat16)
with torch.no_grad():
    want = F.relu(lin(a))
    with dvm.lazy_fusion() as lf:
        got = F.relu(lin(a))
torch.cuda.synchronize()
assert lf.stats["captured"] == 2 and torch.allclose(got.float(), want.float(), rtol=3e-2, atol=3e-2), lf.stats
q, k = rnd(4, 128, 64, dtype=torch.float16), rnd(4, 64, 96, dtype=torch.float16)
with dvm.lazy_fusion() as lf:
    got = torch.bmm(q, k) * 0.125
torch.cuda.synchronize()
assert lf.stats["launches"] == 1 and torch.allclose(got.float(), (torch.bmm(q, k) * 0.125).float(), rtol=1e-2, atol=1e-2)
print("matmul: ok")

# ---- fallbacks keep the program's order: an operator outside the table, an in-place update, a copy to the host ----
x = rnd(64, 1000)
def prog(x):
    x = x.clone()
    a = x * 2.0 + 1.0
    s, _ = torch.sort(a, dim=-1)          # not in the table: a is needed, the segment runs first
    b = s - x
    x.add_(5.0)                            # in place on memory the pending segment reads: the segment runs first
    c = b * x
    return c, float(c.sum().item()), a.cpu()
want = prog(x)
with dvm.lazy_fusion() as lf:
    got = prog(x)
assert torch.allclose(got[0], want[0], rtol=1e-5, atol=1e-5) and abs(got[1] - want[1]) <= 1e-3 * abs(want[1]) + 1e-2 and torch.equal(got[2], want[2].cpu())
assert lf.stats["flushes"] >= 3 and lf.stats["fallbacks"] >= 3, lf.stats
print("fallbacks: ok", lf.stats)

# ---- views: rows at a stride are read in place; a column stride is left to torch ----
big = rnd(200, 512)
with dvm.lazy_fusion() as lf:
    r = big[::2] * 3.0 + big[1::2]
    cvw = big[:, ::2] * 3.0
torch.cuda.synchronize()
assert torch.allclose(r, big[::2] * 3.0 + big[1::2]) and torch.allclose(cvw, big[:, ::2] * 3.0)
assert lf.stats["captured"] == 2, lf.stats
print("views: ok")

# ---- the same sequence again: compiled once ----
lf = dvm.lazy_fusion()
for i in range(4):
    t = rnd(128, 256)
    with lf:
        u = torch.exp(t * 0.5) + 1.0
    torch.cuda.synchronize()
    assert torch.allclose(u, torch.exp(t * 0.5) + 1.0, rtol=1e-6, atol=1e-6)
assert lf.stats["compiled"] == 1 and lf.stats["flushes"] == 4, lf.stats
print("cache: ok")

# ---- a 16-bit tensor and a number: torch computes in fp32 with the number as it is and rounds once ----
for dt in (torch.bfloat16, torch.float16):
    h = rnd(300, 257, dtype=dt)
    def numbers(h):
        return [(h.abs() + 0.6762023455442653) * 0.9084074272936424, 2.0 - h, h / 3.0, F.leaky_relu(h, 0.1), h ** 2,
                torch.where(h > 0.3, h, h * 1.3137085138672244)]
    want = numbers(h)
    with dvm.lazy_fusion() as lf:
        got = numbers(h)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert a.dtype == b.dtype and torch.equal(a, b), (dt, (a.float() - b.float()).abs().max())
print("numbers: ok")

# ---- long expressions are cut into segments; an exception inside the block leaves nothing pending ----
t = rnd(1000)
with dvm.lazy_fusion() as lf:
    v = t
    for i in range(120):
        v = v * 1.01 + 0.001
torch.cuda.synchronize()
w = t
for i in range(120):
    w = w * 1.01 + 0.001
assert torch.allclose(v, w, rtol=1e-4, atol=1e-5) and lf.stats["flushes"] >= 5, lf.stats
try:
    with dvm.lazy_fusion() as lf:
        z = t + 1.0
        raise KeyError("stop")
except KeyError:
    pass
assert lf.stats["flushes"] == 0 and not lf._nodes
print("segments: ok")
'''


def test_lazy_fusion_of_eager_torch_programs():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    done = subprocess.run([sys.executable, "-c", _SCRIPT], cwd=root, env=env, capture_output=True, text=True, timeout=280)
    assert done.returncode == 0, done.stdout + "\n" + done.stderr
    for line in ("example: ok", "activations: ok", "rmsnorm: ok", "matmul: ok", "fallbacks: ok", "views: ok", "cache: ok", "numbers: ok", "segments: ok"):
        assert line in done.stdout, done.stdout + "\n" + done.stderr
