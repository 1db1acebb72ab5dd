"""GPU parity of the LoRA linear (forward and backward) against the CPU oracle.

Tolerance: rel-L2 <= 1e-2 for y, dx, dA, dB against the fp32 oracle evaluated
on the same bf16-valued inputs."""
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import lora_oracle  # noqa: E402

from art_amd import ops  # noqa: E402
from art_amd.lora import LoRALinear, lora_linear  # noqa: E402

pytestmark = pytest.mark.gpu
TOL = 1e-2


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def make(T, n_in, n_out, r, seed, b_std=0.01):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, n_in, generator=g).to(torch.bfloat16)
    W = (0.02 * torch.randn(n_out, n_in, generator=g)).to(torch.bfloat16)
    bound = 1.0 / math.sqrt(n_in)  # Kaiming-uniform with a = sqrt(5)
    A = ((torch.rand(r, n_in, generator=g) * 2 - 1) * bound).to(torch.bfloat16)
    B = (b_std * torch.randn(n_out, r, generator=g)).to(torch.bfloat16)
    up = torch.randn(T, n_out, generator=g).to(torch.bfloat16)
    return x, W, A, B, up


def run_gpu(x, W, A, B, up, scale, gpu):
    xd, Wd, Ad, Bd, upd = (t.to(gpu) for t in (x, W, A, B, up))
    y, xa = ops.lora_linear_fwd(xd, Wd, Ad, Bd, scale)
    dx, dA, dB = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    return y.cpu().float(), dx.cpu().float(), dA.cpu(), dB.cpu()


@pytest.mark.parametrize("T,n_in,n_out,r", [(512, 256, 256, 8), (300, 192, 320, 8), (256, 128, 64, 16),
                                            (1000, 512, 576, 24)])
def test_lora_matches_oracle(artk_lib, gpu, T, n_in, n_out, r):
    print(f"lora T={T} in={n_in} out={n_out} r={r}", flush=True)
    x, W, A, B, up = make(T, n_in, n_out, r, T + r)
    scale = 16 / r
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, scale, up)
    y, dx, dA, dB = run_gpu(x, W, A, B, up, scale, gpu)
    assert rel_l2(y, y0) <= TOL
    assert rel_l2(dx, dx0) <= TOL
    assert rel_l2(dA, dA0) <= TOL
    assert rel_l2(dB, dB0) <= TOL


def test_lora_zero_factors(artk_lib, gpu):
    """B = 0: y is the base projection and dA vanishes; A = 0: dB vanishes."""
    x, W, A, B, up = make(256, 128, 192, 8, 5)
    y, dx, dA, dB = run_gpu(x, W, A, torch.zeros_like(B), up, 2.0, gpu)
    base = ops.gemm_nt(W.to(gpu), x.to(gpu)).cpu().float()
    assert torch.equal(y, base)
    assert dA.abs().max().item() == 0.0
    assert dB.abs().max().item() > 0.0
    y, dx, dA, dB = run_gpu(x, W, torch.zeros_like(A), B, up, 2.0, gpu)
    assert dB.abs().max().item() == 0.0
    assert dA.abs().max().item() > 0.0


@pytest.mark.parametrize("n_out", [2048, 256, 11008])
def test_lora_config2_full_size(artk_lib, gpu, n_out):
    """Benchmark config 2 (Qwen2.5-3B projections) at full size."""
    print(f"lora config2 out={n_out}", flush=True)
    x, W, A, B, up = make(8192, 2048, n_out, 8, 1002 + n_out)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, 2.0, up)
    y, dx, dA, dB = run_gpu(x, W, A, B, up, 2.0, gpu)
    assert rel_l2(y, y0) <= TOL
    assert rel_l2(dx, dx0) <= TOL
    assert rel_l2(dA, dA0) <= TOL
    assert rel_l2(dB, dB0) <= TOL


def test_lora_down_projection_full_size(artk_lib, gpu):
    """The seventh target module of the reference's adapter config (down_proj, 11008 -> 2048,
    src/art/dev/model.py:54-62) at full size, with rank 16."""
    print("lora down_proj 11008 -> 2048, r=16", flush=True)
    x, W, A, B, up = make(4096, 11008, 2048, 16, 1717)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, 1.0, up)
    y, dx, dA, dB = run_gpu(x, W, A, B, up, 1.0, gpu)
    assert rel_l2(y, y0) <= TOL
    assert rel_l2(dx, dx0) <= TOL
    assert rel_l2(dA, dA0) <= TOL
    assert rel_l2(dB, dB0) <= TOL


def test_lora_module_autograd(artk_lib, gpu):
    torch.manual_seed(0)
    mod = LoRALinear(256, 320, r=8, lora_alpha=16, device=gpu, dtype=torch.float32)
    with torch.no_grad():
        mod.lora_B.normal_(std=0.01)
    x = torch.randn(2, 96, 256, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    y = mod(x)
    assert y.shape == (2, 96, 320)
    up = torch.randn_like(y)
    y.backward(up)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(
        x.detach().cpu().view(-1, 256), mod.weight.cpu(), mod.lora_A.detach().cpu().to(torch.bfloat16),
        mod.lora_B.detach().cpu().to(torch.bfloat16), mod.scaling, up.cpu().view(-1, 320))
    assert rel_l2(y.detach().cpu().float().view(-1, 320), y0) <= TOL
    assert rel_l2(x.grad.cpu().float().view(-1, 256), dx0) <= TOL
    assert rel_l2(mod.lora_A.grad.cpu(), dA0) <= TOL
    assert rel_l2(mod.lora_B.grad.cpu(), dB0) <= TOL
    assert mod.weight.grad is None


def test_fused_projections_match_separate(artk_lib, gpu):
    """q/k/v as one product: same outputs and gradients as three LoRALinear modules."""
    from art_amd.lora import FusedLoRALinear, LoRALinear
    torch.manual_seed(5)
    T, n_in = 192, 256
    layers = [LoRALinear(n_in, o, r=8, lora_alpha=16, device=gpu, dtype=torch.float32) for o in (256, 64, 64)]
    for l in layers:
        torch.nn.init.normal_(l.lora_B, std=0.05)
    fused = FusedLoRALinear(layers)
    x1 = torch.randn(T, n_in, device=gpu).to(torch.bfloat16).requires_grad_(True)
    x2 = x1.detach().clone().requires_grad_(True)
    ups = [torch.randn(T, o, device=gpu).to(torch.bfloat16) for o in (256, 64, 64)]
    ys = [l(x1) for l in layers]
    sum((y.float() * u.float()).sum() for y, u in zip(ys, ups)).backward()
    ref = [(l.lora_A.grad.clone(), l.lora_B.grad.clone()) for l in layers]
    for l in layers:
        l.lora_A.grad = None
        l.lora_B.grad = None
    yf = fused(x2)
    sum((y.float() * u.float()).sum() for y, u in zip(yf, ups)).backward()
    rel = lambda a, b: ((a.double() - b.double()).norm() / b.double().norm()).item()
    for a, b in zip(yf, ys):
        assert rel(a.float(), b.float()) <= 4e-3
    assert rel(x2.grad.float(), x1.grad.float()) <= 1e-2
    for l, (dA, dB) in zip(layers, ref):
        assert rel(l.lora_A.grad, dA) <= 1e-2 and rel(l.lora_B.grad, dB) <= 1e-2


@pytest.mark.parametrize("n_out,r", [(2048, 8), (256, 8), (320, 48)])
def test_lora_bias_and_ranks(artk_lib, gpu, n_out, r):
    """Qwen2.5's q/k/v projections carry a (frozen) bias: y = x W^T + bias + s (x A^T) B^T at the
    config-2 q and k/v shapes, and a rank above 32 on a ragged shape (two e tiles in the
    one-pass skinny products).  The bias adds nothing to dx, dA, dB."""
    print(f"lora bias out={n_out} r={r}", flush=True)
    T, n_in = (8192, 2048) if r == 8 else (1100, 448)
    x, W, A, B, up = make(T, n_in, n_out, r, 77 + n_out)
    bias = (0.5 * torch.randn(n_out, generator=torch.Generator().manual_seed(n_out))).to(torch.bfloat16)
    scale = 16 / r
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, scale, up)
    y0 = y0 + bias.float()
    xd, Wd, Ad, Bd, upd = (t.to(gpu) for t in (x, W, A, B, up))
    y, xa = ops.lora_linear_fwd(xd, Wd, Ad, Bd, scale, bias.to(gpu))
    dx, dA, dB = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL
    # bit-reproducible run to run (fixed summation orders)
    dx2, dA2, dB2 = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    assert torch.equal(dA, dA2) and torch.equal(dB, dB2) and torch.equal(dx, dx2)


def test_lora_module_with_bias_from_linear(artk_lib, gpu):
    """LoRALinear.from_linear keeps the base layer's bias (as peft does) and leaves it frozen."""
    torch.manual_seed(3)
    lin = torch.nn.Linear(256, 192, bias=True, device=gpu, dtype=torch.bfloat16)
    mod = LoRALinear.from_linear(lin, r=8, lora_alpha=16)
    assert mod.bias is not None and not mod.bias.requires_grad
    with torch.no_grad():
        mod.lora_B.normal_(std=0.02)
    x = torch.randn(300, 256, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    y = mod(x)
    y.backward(torch.ones_like(y))
    want = (x.detach().float() @ lin.weight.float().t() + lin.bias.float()
            + mod.scaling * (x.detach().float() @ mod.lora_A.float().t()) @ mod.lora_B.float().t())
    assert rel_l2(y.detach().float().cpu(), want.cpu()) <= TOL
    assert mod.bias.grad is None and mod.lora_A.grad is not None
