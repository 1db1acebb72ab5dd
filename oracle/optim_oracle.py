"""CPU oracle of the optimizer step.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference configures HF Trainer with AdamW (`paged_adamw_8bit`), betas
(0.9, 0.99), weight_decay 0.1, max_grad_norm 0.1 (src/art/dev/model.py:69-85);
the update itself is library code.  The oracle is torch's own
`torch.optim.AdamW` preceded by `torch.nn.utils.clip_grad_norm_` on CPU fp32
tensors (library routines, so nothing is restated here); the 8-bit block-wise
quantisation of the moments done by bitsandbytes is not modelled: PARITY
UNPINNED against bitsandbytes (absent)."""
from __future__ import annotations

import torch


def adamw_steps(p0, grads, lr, betas, eps, weight_decay, max_grad_norm):
    """Apply one AdamW step per gradient in `grads` to a copy of p0; returns
    (params, exp_avg, exp_avg_sq, [squared norms before clipping])."""
    p = torch.nn.Parameter(p0.clone().float())
    opt = torch.optim.AdamW([p], lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, foreach=False)
    norms = []
    for g in grads:
        p.grad = g.clone().float()
        if max_grad_norm:
            n = torch.nn.utils.clip_grad_norm_([p], max_grad_norm)
            norms.append(float(n) ** 2)
        else:
            norms.append(float(p.grad.double().pow(2).sum()))
        opt.step()
    st = opt.state[p]
    return p.detach(), st["exp_avg"], st["exp_avg_sq"], norms
