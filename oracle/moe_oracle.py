"""CPU oracle of the MoE expert path.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference has no MoE code at this commit, so there is nothing of its own to
restate: PARITY UNPINNED against the reference.  The contract is the benchmark
configuration plus the usual definitions, stated here with plain torch:
  routing      softmax over router logits in fp32, top-k, renormalise (the
               semantics of transformers' Qwen3-MoE block); selection on the
               logits, ties to the lower expert index; a NaN logit counts as
               -inf, an expert at -inf gets weight 0, a row without a finite
               logit gets weights 0
  permutation  stable sort of the token-major (token, slot) list by expert id
  projections  per expert y = x W_e^T + scale (x A_e^T) B_e^T  (Python loop)
Pinned in tests/test_oracle_moe.py by brute force on tiny inputs, by
torch.topk / torch.sort(stable=True) as library routines, and by invariants
(perm is a permutation, rows of an expert are contiguous and in token order)."""
from __future__ import annotations

import torch


def route(router_logits: torch.Tensor, k: int):
    """Returns dict(topk_idx [T,k], topk_w [T,k], perm [T*k], inv_perm, row_token, offsets [E+1])."""
    T, E = router_logits.shape
    logits = router_logits.float()
    # NaN counts as -inf (a masked expert); the order is then total
    logits = torch.where(torch.isnan(logits), torch.full_like(logits, float("-inf")), logits)
    order = torch.sort(-logits, dim=-1, stable=True).indices  # ties -> lower index first
    topk_idx = order[:, :k]
    # softmax mass of the chosen experts; exp(-inf - m) = 0, and a row without any finite
    # logit carries no mass at all (its weights are 0 rather than NaN)
    m = logits.max(-1, keepdim=True).values
    chosen = logits.gather(-1, topk_idx)
    p = torch.where(torch.isinf(chosen) & (chosen < 0), torch.zeros_like(chosen), torch.exp(chosen - m))
    tot = p.sum(-1, keepdim=True)
    topk_w = torch.where(tot > 0, p / tot, torch.zeros_like(p))
    flat = topk_idx.reshape(-1)
    perm = torch.sort(flat, stable=True).indices
    inv_perm = torch.empty_like(perm)
    inv_perm[perm] = torch.arange(perm.numel())
    counts = torch.bincount(flat, minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int64)
    offsets[1:] = counts.cumsum(0)
    return {"topk_idx": topk_idx, "topk_w": topk_w, "perm": perm, "inv_perm": inv_perm,
            "row_token": perm // k, "offsets": offsets}


def grouped_lora(x_rows, W, A, B, scale, offsets):
    """y[i] = x_rows[i] W_e^T + scale (x_rows[i] A_e^T) B_e^T for the rows i of expert e."""
    out = []
    for e in range(W.shape[0]):
        xs = x_rows[offsets[e]:offsets[e + 1]]
        out.append(xs @ W[e].t() + scale * ((xs @ A[e].t()) @ B[e].t()))
    return torch.cat(out, 0)


def grouped_lora_grads(x, row_token, W, A, B, scale, offsets, g, dtype=torch.float32):
    """(y, dx [like x], dA, dB) by autograd; row_token None means x is already in sorted row order."""
    x_ = x.to(dtype).clone().requires_grad_(True)
    A_ = A.to(dtype).clone().requires_grad_(True)
    B_ = B.to(dtype).clone().requires_grad_(True)
    rows = x_ if row_token is None else x_[row_token]
    y = grouped_lora(rows, W.to(dtype), A_, B_, scale, offsets)
    y.backward(g.to(dtype))
    return y.detach(), x_.grad, A_.grad, B_.grad
