"""Writes tests/golden/grpo_small.npz: one small GRPO case with its inputs (bit patterns of
the bf16 tensors, so nothing depends on a random generator) and the values the float64
evaluation of the reference's formulas gives for them.

The reference ships no vectors of its own for this path; these are frozen outputs of this
repository's CPU restatement, evaluated here in float64 with plain torch routines
(log_softmax, autograd) following src/art/local/train.py:111-151, 245-285.  They guard
the oracle and the kernels against drifting together; what pins the formulas themselves
is in tests/test_oracle_grpo.py.

Run from the repository root:  python tests/golden/make_grpo_fixture.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from art_amd import synthetic  # noqa: E402


def shift(t, pad):
    return torch.cat([t[:, 1:], torch.full_like(t[:, :1], pad)], 1)


def main():
    T, H, V = 256, 64, 1024
    case = synthetic.make_grpo_case("golden", 4242, T, H, V, 4, 4, 0.5)
    hidden = case.hidden.double().requires_grad_(True)            # [1, T, H]
    W = case.lm_head.double()                                     # [V, H]
    nxt = shift(case.tokens, 0)
    logits = hidden @ W.t()
    new = torch.log_softmax(logits, -1).gather(-1, nxt.unsqueeze(-1)).squeeze(-1)
    case.finish(new.detach().float())
    old = shift(case.logprobs, 0.0).double()
    adv = shift(case.advantages, 0.0).double()
    mask = shift(case.assistant_mask, False).double()
    w = shift(case.weights, 0.0).double()
    old = torch.where(torch.isnan(old), new.detach(), old)
    ratio = torch.exp(new - old)
    eps = 0.2
    pl = -torch.minimum(ratio * adv, torch.clip(ratio, 1 - eps, 1 + eps) * adv) * w * mask
    loss = pl.sum() / (mask.sum() + 1e-6)
    loss.backward()
    bits = lambda t: t.contiguous().view(torch.int16).numpy()
    np.savez_compressed(
        os.path.join(os.path.dirname(os.path.abspath(__file__)), "grpo_small.npz"),
        hidden_bits=bits(case.hidden), lm_head_bits=bits(case.lm_head), tokens=case.tokens.numpy(),
        logprobs=case.logprobs.numpy(), advantages=case.advantages.numpy(),
        assistant_mask=case.assistant_mask.numpy(), weights=case.weights.numpy(),
        epsilon=np.float64(eps),
        expect_new_logprobs=new.detach().float().numpy(), expect_loss=np.float64(loss.item()),
        expect_loss_abs_terms=np.float64((pl.abs().sum() / (mask.sum() + 1e-6)).item()),
        expect_mask_count=np.float64(mask.sum().item()), expect_d_hidden=hidden.grad.float().numpy())
    print("loss", loss.item(), "mask", mask.sum().item())


if __name__ == "__main__":
    main()
