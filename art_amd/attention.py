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

import torch.nn.functional as F

from . import ops

ROW_MULTIPLE = 256  # the kernels take rows whose length is a multiple of this


def attention_plans(group_ids: torch.Tensor, parent_ids: torch.Tensor) -> List[ops.AttnPlan]:
    """One plan per packed row of ``group_ids`` / ``parent_ids`` ([B, S] int64, the
    PackedTensors rows of src/art/local/pack.py:13-21).  Make them once per
    batch; every layer and head reuses them."""
    if group_ids.dim() == 1:
        group_ids, parent_ids = group_ids.unsqueeze(0), parent_ids.unsqueeze(0)
    S = group_ids.shape[1]
    extra = -S % ROW_MULTIPLE
    if extra:
        # Rows of any length: append positions whose ids no real position carries (as group
        # or as parent), so they see and are seen by nothing but themselves; packed_attention
        # pads q, k, v to match and drops their outputs.
        fill = (torch.minimum(group_ids.amin(), parent_ids.amin()) - 1).reshape(1, 1)
        fill = fill.expand(group_ids.shape[0], extra)
        group_ids = torch.cat([group_ids, fill], 1)
        parent_ids = torch.cat([parent_ids, fill], 1)
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
        return _row(q, k, v, plans[0], scale)
    outs = [_row(q[b], k[b], v[b], plans[b], scale) for b in range(q.shape[0])]
    return torch.stack(outs, 0)


def _row(q, k, v, plan, scale):
    S = q.shape[0]
    extra = plan.S - S
    if extra == 0:
        return _PackedAttentionFn.apply(q, k, v, plan, scale)
    if not 0 < extra < ROW_MULTIPLE:
        raise ValueError(f"plan made for a row of {plan.S} positions, tensors have {S}")
    if scale is None:
        scale = float(q.shape[-1]) ** -0.5
    pad = (0, 0, 0, 0, 0, extra)  # zero rows at the end of the sequence dimension
    out = _PackedAttentionFn.apply(F.pad(q, pad), F.pad(k, pad), F.pad(v, pad), plan, scale)
    return out[:S]
