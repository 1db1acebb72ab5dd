"""CPU oracle of the MoE expert path.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference has no MoE code at this commit, so there is nothing of its own to
restate: PARITY UNPINNED against the reference.  The contract is the benchmark
configuration plus the usual definitions, stated here with plain torch:
  routing      softmax over router logits in fp32, top-k, renormalise (the
               semantics of transformers' Qwen3-MoE block); selection on the
               logits, ties to the lower expert index
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
    probs = torch.softmax(logits, dim=-1)
    order = torch.sort(-logits, dim=-1, stable=True).indices  # ties -> lower index first
    topk_idx = order[:, :k]
    p = probs.gather(-1, topk_idx)
    topk_w = p / p.sum(-1, keepdim=True)
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
