"""CPU oracle of the packed-row attention.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference builds a dense additive bias from the packed row's group and
parent ids (src/art/local/train.py:177-215):

    visible(i, j) = j <= i  and  (group[i] == group[j]  or  parent[i] == group[j])
    bias = 0 where visible else -inf

and hands it to the model as `causal_mask` (train.py:239-241); the attention
that consumes it lives in the third-party model code (transformers / unsloth,
not in the reference tree) and is the textbook softmax(Q K^T / sqrt(d) + bias) V
with grouped-query heads.  `visibility` is pinned by a brute-force double loop
on tiny id arrays and `attention` against torch's own
scaled_dot_product_attention with the same mask (tests/test_oracle_attn.py);
the third-party attention itself is PARITY UNPINNED (no fixture of it exists).
"""
from __future__ import annotations

import math

import torch


def visibility(group_ids: torch.Tensor, parent_ids: torch.Tensor) -> torch.Tensor:
    """bool [B, S, S] following train.py:185-199 (tril & (group | parent))."""
    S = group_ids.shape[-1]
    causal = torch.tril(torch.ones(S, S, dtype=torch.bool)).unsqueeze(0)
    group = group_ids.unsqueeze(2) == group_ids.unsqueeze(1)
    parent = parent_ids.unsqueeze(2) == group_ids.unsqueeze(1)
    return causal & (group | parent)


def attn_bias(group_ids, parent_ids, dtype=torch.float32) -> torch.Tensor:
    """Additive bias [B, S, S]: 0 where visible, -inf elsewhere (train.py:200-215)."""
    vis = visibility(group_ids, parent_ids)
    return torch.where(vis, torch.zeros((), dtype=dtype), torch.full((), float("-inf"), dtype=dtype))


def attention(q, k, v, group_ids, parent_ids, scale=None, dtype=torch.float32):
    """q [S, Hq, D], k/v [S, Hkv, D], ids [S] -> (out [S, Hq, D], lse [Hq, S]) in `dtype`.

    Query head h uses key/value head h // (Hq // Hkv)."""
    S, Hq, D = q.shape
    Hkv = k.shape[1]
    rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    bias = attn_bias(group_ids.view(1, S), parent_ids.view(1, S), dtype)[0]
    qh = q.to(dtype).permute(1, 0, 2)                              # [Hq, S, D]
    kh = k.to(dtype).permute(1, 0, 2).repeat_interleave(rep, 0)    # [Hq, S, D]
    vh = v.to(dtype).permute(1, 0, 2).repeat_interleave(rep, 0)
    s = qh @ kh.transpose(1, 2) * scale + bias
    lse = torch.logsumexp(s, -1)
    p = torch.exp(s - lse.unsqueeze(-1))
    out = (p @ vh).permute(1, 0, 2)
    return out, lse


def attention_grads(q, k, v, group_ids, parent_ids, d_out, scale=None, dtype=torch.float32):
    """(out, dq, dk, dv) by autograd in `dtype` on up-casts of the inputs."""
    q_ = q.to(dtype).clone().requires_grad_(True)
    k_ = k.to(dtype).clone().requires_grad_(True)
    v_ = v.to(dtype).clone().requires_grad_(True)
    out, _ = attention(q_, k_, v_, group_ids, parent_ids, scale, dtype)
    out.backward(d_out.to(dtype))
    return out.detach(), q_.grad, k_.grad, v_.grad


def visible_pairs(group_ids, parent_ids) -> int:
    """Number of (query, key) pairs the bias leaves visible in one row."""
    S = group_ids.numel()
    return int(visibility(group_ids.view(1, S), parent_ids.view(1, S)).sum().item())


def attention_rows(q, k, v, group_ids, parent_ids, rows, scale=None, dtype=torch.float32):
    """Same as `attention` for the query positions `rows` (1-D index tensor) only:
    out [len(rows), Hq, D], lse [Hq, len(rows)].  For sizes where the S x S bias
    does not fit; the rule is the one of train.py:185-199 applied to the window."""
    S, Hq, D = q.shape
    Hkv = k.shape[1]
    rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    dev = q.device  # all inputs on one device (the full-size tests run this restatement on the GPU)
    j = torch.arange(S, device=dev).unsqueeze(0)
    vis = (j <= rows.unsqueeze(1)) & ((group_ids[rows].unsqueeze(1) == group_ids.unsqueeze(0)) |
                                      (parent_ids[rows].unsqueeze(1) == group_ids.unsqueeze(0)))
    bias = torch.where(vis, torch.zeros((), dtype=dtype, device=dev),
                       torch.full((), float("-inf"), dtype=dtype, device=dev))
    qh = q[rows].to(dtype).permute(1, 0, 2)
    kh = k.to(dtype).permute(1, 0, 2).repeat_interleave(rep, 0)
    vh = v.to(dtype).permute(1, 0, 2).repeat_interleave(rep, 0)
    s = qh @ kh.transpose(1, 2) * scale + bias
    lse = torch.logsumexp(s, -1)
    out = (torch.exp(s - lse.unsqueeze(-1)) @ vh).permute(1, 0, 2)
    return out, lse
