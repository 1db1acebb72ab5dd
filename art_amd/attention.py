"""Attention over a packed row without the dense bias.

The reference builds ``attn_bias = calculate_attn_bias(...)`` ([B, S, S], 0 / -inf)
and passes it to the model as ``causal_mask`` (src/art/local/train.py:66-73,
177-215, 239-241).  ``packed_attention`` is what a model's attention layer calls
instead of ``softmax(q k^T * scale + attn_bias) v``: same inputs minus the bias,
plus the two id rows the bias was made from.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from . import ops


def attention_plans(group_ids: torch.Tensor, parent_ids: torch.Tensor) -> List[ops.AttnPlan]:
    """One plan per packed row of ``group_ids`` / ``parent_ids`` ([B, S] int64, the
    PackedTensors rows of src/art/local/pack.py:13-21).  Make them once per
    batch; every layer and head reuses them."""
    if group_ids.dim() == 1:
        group_ids, parent_ids = group_ids.unsqueeze(0), parent_ids.unsqueeze(0)
    return [ops.attn_plan(g.contiguous(), p.contiguous()) for g, p in zip(group_ids, parent_ids)]


class _PackedAttentionFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, plan, scale):
        out, lse = ops.attn_fwd(q, k, v, plan, scale)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.plan, ctx.scale = plan, scale
        return out

    @staticmethod
    def backward(ctx, d_out):
        q, k, v, out, lse = ctx.saved_tensors
        if d_out.stride(2) != 1:
            d_out = d_out.contiguous()
        dq, dk, dv = ops.attn_bwd(q, k, v, out, lse, d_out.to(torch.bfloat16), ctx.plan, ctx.scale)
        return dq, dk, dv, None, None


def packed_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, plans: List[ops.AttnPlan],
                     scale: Optional[float] = None) -> torch.Tensor:
    """softmax(q k^T * scale + bias) v with the bias of calculate_attn_bias, never built.

    q [B, S, Hq, D], k / v [B, S, Hkv, D] bf16 (any strides over B, S, H; D contiguous;
    a [B, H, S, D] tensor goes in as ``t.transpose(1, 2)``).  Returns [B, S, Hq, D] bf16.
    Differentiable w.r.t. q, k, v."""
    if q.dim() == 3:
        return _PackedAttentionFn.apply(q, k, v, plans[0], scale)
    outs = [_PackedAttentionFn.apply(q[b], k[b], v[b], plans[b], scale) for b in range(q.shape[0])]
    return torch.stack(outs, 0)
