"""CPU oracle of the optimizer step.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference configures HF Trainer with AdamW (`paged_adamw_8bit`), betas
(0.9, 0.99), weight_decay 0.1, max_grad_norm 0.1 (src/art/dev/model.py:69-85);
the update itself is library code.  The oracle is torch's own
`torch.optim.AdamW` preceded by `torch.nn.utils.clip_grad_norm_` on CPU fp32
tensors (library routines, so nothing is restated here).

`adamw8bit_step` restates the block-wise 8-bit form of the moments that
`paged_adamw_8bit` uses (bitsandbytes, absent: PARITY UNPINNED against that
package; restated from the published method, Dettmers et al. 2022, and its
public kernel's update order).  Pinned in tests/test_oracle_optim.py: quantising a
code book entry gives that entry back; the first step from zero state equals the
closed form up to the code book's resolution; after many steps the parameters
track torch.optim.AdamW within the quantisation error."""
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


def nearest_code(book, x):
    """Index of the entry of the ascending `book` nearest to each x (ties to the lower index)."""
    import numpy as np

    book = np.asarray(book, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    hi = np.clip(np.searchsorted(book, x, side="right"), 1, 255)   # first entry > x
    # searchsorted(side=right) - 1 is the last entry <= x; with duplicates (padding zeros) the
    # kernel's bisection also ends on the last of them
    lo = hi - 1
    take_lo = (x - book[lo]) <= (book[hi] - x)
    return np.where(take_lo, lo, hi).astype(np.uint8)


def adamw8bit_step(p, g, c1, c2, absmax1, absmax2, book1, book2, lr, betas, eps, weight_decay, step,
                   max_grad_norm=0.0):
    """One step on float32 / uint8 numpy arrays (n a multiple of 256 or padded by the caller);
    returns new (p, c1, c2, absmax1, absmax2).  Every operation is a single float32 operation
    in the order of the kernel."""
    import numpy as np

    f = np.float32
    p, g = np.asarray(p, f), np.asarray(g, f)
    n = p.size
    nb = (n + 255) // 256
    clip = f(1.0)
    if max_grad_norm:
        c = f(max_grad_norm) / (np.sqrt(f(np.sum(g.astype(np.float64) ** 2))) + f(1e-6))
        clip = f(min(c, f(1.0)))
    g = g * clip
    b1, b2 = f(betas[0]), f(betas[1])
    blk = np.arange(n) // 256
    m = np.asarray(book1, f)[c1] * np.asarray(absmax1, f)[blk]
    v = np.asarray(book2, f)[c2] * np.asarray(absmax2, f)[blk]
    m = m * b1 + (f(1.0) - b1) * g
    v = v * b2 + ((f(1.0) - b2) * g) * g
    pad = nb * 256 - n
    mx1 = np.abs(np.pad(m, (0, pad))).reshape(nb, 256).max(1).astype(f)
    mx2 = np.abs(np.pad(v, (0, pad))).reshape(nb, 256).max(1).astype(f)
    corr1 = 1.0 - betas[0] ** step
    corr2 = (1.0 - betas[1] ** step) ** 0.5
    step_size = f(-lr * corr2 / corr1)
    p = p + step_size * (m / (np.sqrt(v) + f(corr2 * eps)))
    if weight_decay > 0:
        p = p * (f(1.0) - f(lr) * f(weight_decay))
    s1 = np.where(mx1[blk] > 0, m / np.where(mx1[blk] > 0, mx1[blk], f(1)), f(0)).astype(f)
    s2 = np.where(mx2[blk] > 0, v / np.where(mx2[blk] > 0, mx2[blk], f(1)), f(0)).astype(f)
    return p.astype(f), nearest_code(book1, s1), nearest_code(book2, s2), mx1, mx2
