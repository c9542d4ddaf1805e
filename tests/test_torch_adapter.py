"""GPU: `@kernel` functions called with torch tensors (the custom fused operator route of the reference's
docs/pytorch.md): inputs are read in place, outputs are torch tensors, launches go to torch's current stream."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_kernel_on_torch_tensors():
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


def test_kernel_runs_on_the_current_torch_stream():
    import torch
    import dvm_amd as dvm

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


def test_kernel_rejects_wrong_tensor_types():
    import torch
    import dvm_amd as dvm

    @dvm.kernel(ktype="vector", dynamic=True)
    def twice(k, x):
        return k.store(k.mul(k.load(x, dvm.float32), 2.0))

    with pytest.raises(TypeError):
        twice(torch.zeros(8, device="cuda", dtype=torch.float16))
    assert np.allclose(twice(np.ones(8, np.float32)), 2.0)  # the numpy route still works on the same kernel
