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


def test_adamw8bit_matches_oracle(artk_lib, gpu):
    """8-bit block-wise moments: five steps against the numpy restatement.  The arithmetic is the
    same float32 operations; the compiler may fuse a multiply-add, so a value that sits on the
    boundary between two codes can fall on the other side: codes must agree on 99.9 % of the
    elements and never differ by more than one, parameters to 1e-6 relative."""
    import numpy as np

    from art_amd.optim import FusedAdamW8bit, dynamic_code_book

    print("adamw 8-bit", flush=True)
    g = torch.Generator().manual_seed(13)
    shapes = {"A0": (8, 2048), "B0": (2048, 8), "A1": (8, 37), "odd": (13,)}
    flat = FlatParams(shapes, gpu)
    flat.master.copy_(torch.randn(flat.numel, generator=g) * 0.05)
    n = flat.numel
    p = flat.master.cpu().numpy().copy()
    grads = [torch.randn(n, generator=g) * (0.5 if i % 2 else 0.01) for i in range(5)]
    lr, wd, eps, betas, clip = 1e-3, 0.1, 1e-8, (0.9, 0.99), 0.1
    opt = FusedAdamW8bit(flat, lr=lr, betas=betas, eps=eps, weight_decay=wd, max_grad_norm=clip)
    b1, b2 = dynamic_code_book(True).numpy(), dynamic_code_book(False).numpy()
    nb = (n + 255) // 256
    c1 = c2 = np.zeros(n, np.uint8)
    a1 = a2 = np.zeros(nb, np.float32)
    for t, gr in enumerate(grads, 1):
        flat.grad.copy_(gr)
        opt.step()
        p, c1, c2, a1, a2 = optim_oracle.adamw8bit_step(p, gr.numpy(), c1, c2, a1, a2, b1, b2, lr, betas, eps,
                                                        wd, t, clip)
        # continue the oracle from the kernel's own stored state, so that one flipped code
        # does not compound over the steps
        got1, got2 = opt.state1.cpu().numpy(), opt.state2.cpu().numpy()
        d1 = np.abs(got1.astype(int) - c1.astype(int))
        d2 = np.abs(got2.astype(int) - c2.astype(int))
        assert (d1 == 0).mean() >= 0.999 and (d2 == 0).mean() >= 0.999 and d1.max() <= 1 and d2.max() <= 1, t
        assert np.allclose(opt.absmax1.cpu().numpy(), a1, rtol=2e-6, atol=0)
        assert np.allclose(opt.absmax2.cpu().numpy(), a2, rtol=2e-6, atol=0)
        got_p = flat.master.cpu().numpy()
        assert np.abs(got_p - p).max() <= 1e-6 * np.abs(p).max(), t
        c1, c2, a1, a2, p = got1, got2, opt.absmax1.cpu().numpy(), opt.absmax2.cpu().numpy(), got_p
    assert torch.equal(flat.shadow, flat.master.to(torch.bfloat16))
    assert opt.exp_avg().shape == (n,) and opt.exp_avg_sq().min().item() >= 0.0
