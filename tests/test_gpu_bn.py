"""Batch normalisation (+ ReLU) kernels of include/phx_bn.h against torch's batch_norm evaluated in fp64 on
the CPU from the same (fp16- or fp32-rounded) inputs: output, saved and running statistics, input gradient
and parameter gradients.  Tolerance: 1e-4 (fp32 tensors) / 4e-3 (fp16 tensors, whose outputs are rounded to
fp16) of the largest reference magnitude."""
import numpy as np
import pytest
import torch

import phoenix_core_amd as phx

pytestmark = pytest.mark.gpu

SHAPES = [(8, 16, 14, 14), (12, 5, 7, 7), (3, 130, 1, 1), (64, 33, 9, 5), (1, 4, 3, 3), (256, 16, 28, 28), (40, 512, 7, 7)]


def close(got, want, tol, what):
    got = got.detach().double().cpu()
    err = (got - want).abs().max().item()
    assert torch.isfinite(got).all(), what
    assert err <= tol * max(want.abs().max().item(), 1e-6), "%s: abs err %.3e of max %.3e" % (what, err, want.abs().max().item())


@pytest.mark.parametrize("relu,residual", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_batch_norm_matches_torch(shape, dtype, relu, residual):
    print("shape", shape, dtype, relu, residual, flush=True)
    gen = torch.Generator().manual_seed(sum(shape))
    c = shape[1]
    x = (torch.randn(shape, generator=gen) * 1.5 + 0.3).to(dtype)
    dy = torch.randn(shape, generator=gen).to(dtype)
    gamma = torch.rand(c, generator=gen) + 0.5
    beta = torch.randn(c, generator=gen) * 0.3
    mod = phx.QBatchNorm2d(c, relu=relu).cuda().train()
    with torch.no_grad():
        mod.weight.copy_(gamma)
        mod.bias.copy_(beta)
    res = (torch.randn(shape, generator=gen) * 0.7).to(dtype) if residual else None
    if relu:
        # The gradient of the ReLU jumps at zero: an element whose pre-activation is zero to rounding error gets its
        # gradient in one precision and not in the other.  Those elements carry no output gradient here.
        with torch.no_grad():
            z = torch.nn.functional.batch_norm(x.double(), None, None, gamma.double(), beta.double(), True, 0.1, 1e-5)
            if residual:
                z = z + res.double()
            dy[z.abs() < (1e-4 if dtype == torch.float32 else 2e-2)] = 0
    xd = x.cuda().requires_grad_(True)
    rd = res.cuda().requires_grad_(True) if residual else None
    y = mod(xd, rd) if residual else mod(xd)
    y.backward(dy.cuda())

    x64 = x.double().requires_grad_(True)
    g64, b64 = gamma.double().requires_grad_(True), beta.double().requires_grad_(True)
    rm, rv = torch.zeros(c, dtype=torch.float64), torch.ones(c, dtype=torch.float64)
    ref = torch.nn.functional.batch_norm(x64, rm, rv, g64, b64, True, 0.1, 1e-5)
    r64 = res.double().requires_grad_(True) if residual else None
    if residual:
        ref = ref + r64
    if relu:
        ref = torch.relu(ref)
    ref.backward(dy.double())
    tol = 1e-4 if dtype == torch.float32 else 4e-3
    assert y.dtype == dtype and y.shape == tuple(shape)
    close(y, ref.detach(), tol, "y")
    close(xd.grad, x64.grad, tol, "dx")
    if residual:
        close(rd.grad, r64.grad, tol, "dresidual")
    close(mod.weight.grad, g64.grad, tol, "dgamma")
    close(mod.bias.grad, b64.grad, tol, "dbeta")
    close(mod.running_mean, rm, 1e-4, "running mean")
    close(mod.running_var, rv, 1e-4, "running var")


def test_eval_mode_uses_running_statistics():
    mod = phx.QBatchNorm2d(6, relu=True).cuda()
    x = torch.randn(8, 6, 5, 5, device="cuda")
    mod.train()
    mod(x)
    mod.eval()
    y = mod(x)
    want = torch.relu(torch.nn.functional.batch_norm(x, mod.running_mean, mod.running_var, mod.weight, mod.bias, False, 0.0,
                                                     mod.eps))
    assert torch.allclose(y, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_statistics_of_a_channel_with_a_large_mean(dtype):
    """Channels whose mean is ~1000 times their spread (fp32) / ~100 times (fp16): E[x^2] - E[x]^2 in fp32 would
    lose every significant bit of the variance; the kernels sum around a shift inside the data's range instead.
    Saved inverse standard deviation, running variance and the normalised output against fp64."""
    gen = torch.Generator().manual_seed(77)
    shape = (32, 6, 12, 12)
    big = 1000.0 if dtype == torch.float32 else 100.0
    offsets = torch.tensor([big, -big, 0.0, 3 * big, big, -2 * big]).view(1, 6, 1, 1)
    x = (torch.randn(shape, generator=gen) + offsets).to(dtype)
    mod = phx.QBatchNorm2d(6, relu=False).cuda().train()
    y = mod(x.cuda())
    x64 = x.double()
    var = x64.var(dim=(0, 2, 3), unbiased=False)
    want = (x64 - x64.mean(dim=(0, 2, 3), keepdim=True)) / (var.view(1, 6, 1, 1) + 1e-5).sqrt()
    n = shape[0] * shape[2] * shape[3]
    close(mod.running_var, 0.9 + 0.1 * var * n / (n - 1), 1e-3, "running var")
    close(y, want, 1e-3 if dtype == torch.float32 else 4e-3, "y")
