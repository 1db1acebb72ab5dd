"""GPU parity of the fused AdamW step against torch.optim.AdamW + clip_grad_norm_
on the CPU (fp32).  Tolerance 2e-6 relative on parameters and moments after five
steps: the update is the same fp32 arithmetic up to the order of a few roundings."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import optim_oracle  # noqa: E402

from art_amd import ops  # noqa: E402
from art_amd.optim import FlatParams, FusedAdamW  # noqa: E402

pytestmark = pytest.mark.gpu


def rel(a, b):
    return ((a.double() - b.double()).abs().max() / b.double().abs().max()).item()


@pytest.mark.parametrize("n", [1, 7, 4096, 1_000_003])
def test_sumsq(artk_lib, gpu, n):
    x = torch.randn(n, generator=torch.Generator().manual_seed(n))
    got = ops.sumsq(x.to(gpu)).item()
    want = x.double().pow(2).sum().item()
    assert abs(got - want) <= 1e-6 * want
    assert ops.sumsq(x.to(gpu)).item() == got  # fixed order


@pytest.mark.parametrize("clip", [0.1, 0.0])
@pytest.mark.parametrize("lr,wd", [(5e-6, 0.1), (1e-2, 0.0)])
def test_adamw_matches_torch(artk_lib, gpu, clip, lr, wd):
    g = torch.Generator().manual_seed(3)
    shapes = {"A0": (8, 100), "B0": (100, 8), "A1": (8, 37), "B1": (37, 8), "odd": (13,)}
    flat = FlatParams(shapes, gpu)
    flat.master.copy_(torch.randn(flat.numel, generator=g) * 0.05)
    p0 = flat.master.cpu().clone()
    grads = [torch.randn(flat.numel, generator=g) * (0.5 if i % 2 else 0.01) for i in range(5)]
    opt = FusedAdamW(flat, lr=lr, betas=(0.9, 0.99), eps=1e-8, weight_decay=wd, max_grad_norm=clip)
    norms = []
    for gr in grads:
        flat.grad.copy_(gr)
        norms.append(opt.step().item())
    ref_p, ref_m, ref_v, ref_norms = optim_oracle.adamw_steps(p0, grads, lr, (0.9, 0.99), 1e-8, wd, clip)
    for a, b in zip(norms, ref_norms):
        assert abs(a - b) <= 1e-5 * b
    assert rel(flat.master.cpu(), ref_p) <= 2e-6
    assert rel(opt.exp_avg.cpu(), ref_m) <= 2e-6
    assert rel(opt.exp_avg_sq.cpu(), ref_v) <= 2e-6
    # the bf16 copy is the rounded master copy, and the named views alias the flat buffers
    assert torch.equal(flat.shadow, flat.master.to(torch.bfloat16))
    assert flat.param("B1").data_ptr() == flat.master.data_ptr() + 4 * flat.offsets["B1"][0]
    assert flat.bf16("A1").shape == (8, 37)
