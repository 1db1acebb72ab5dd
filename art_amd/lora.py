"""LoRA linear layer on the MI355X kernels.

``LoRALinear`` is the counterpart of the peft ``lora.Linear`` module that the
reference installs on the attention and MLP projections
(src/art/local/state.py:86-92; defaults r = 8, alpha = 16, no dropout, no bias:
src/art/dev/model.py:52-67).  The base weight is frozen; only ``lora_A`` and
``lora_B`` receive gradients."""
from __future__ import annotations

import math

import torch
from torch import nn

from . import ops


class _LoRALinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, lora_A, lora_B, scale):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).to(torch.bfloat16).contiguous()
        A = lora_A.detach().to(torch.bfloat16).contiguous()
        B = lora_B.detach().to(torch.bfloat16).contiguous()
        y, xa = ops.lora_linear_fwd(x2, weight, A, B, scale)
        ctx.save_for_backward(x2, weight, A, B, xa)
        ctx.scale = scale
        ctx.lead = lead
        ctx.param_dtypes = (lora_A.dtype, lora_B.dtype, x.dtype)
        return y.view(*lead, weight.shape[0])

    @staticmethod
    def backward(ctx, g):
        x2, weight, A, B, xa = ctx.saved_tensors
        g2 = g.reshape(-1, g.shape[-1]).to(torch.bfloat16).contiguous()
        dx, dA, dB = ops.lora_linear_bwd(g2, x2, ops.transposed_weight(weight), A, B, xa, ctx.scale)
        a_dtype, b_dtype, x_dtype = ctx.param_dtypes
        return (dx.view(*ctx.lead, x2.shape[-1]).to(x_dtype), None, dA.to(a_dtype), dB.to(b_dtype), None)


def lora_linear(x, weight, lora_A, lora_B, scale: float):
    """y = x W^T + scale * (x A^T) B^T with gradients for x, A and B (W frozen)."""
    return _LoRALinearFn.apply(x, weight, lora_A, lora_B, float(scale))


class LoRALinear(nn.Module):
    """Frozen bf16 linear with a trainable rank-r update; forward(x) -> y."""

    def __init__(self, in_features: int, out_features: int, r: int = 8, lora_alpha: int = 16,
                 device=None, dtype=torch.bfloat16):
        super().__init__()
        self.in_features, self.out_features, self.r = in_features, out_features, r
        self.scaling = lora_alpha / r
        self.weight = nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=torch.bfloat16),
                                   requires_grad=False)
        self.lora_A = nn.Parameter(torch.empty(r, in_features, device=device, dtype=dtype))
        self.lora_B = nn.Parameter(torch.zeros(out_features, r, device=device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, std=0.02)
        nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))  # peft's default for A; B starts at zero
        nn.init.zeros_(self.lora_B)

    @classmethod
    def from_linear(cls, linear: nn.Linear, r: int = 8, lora_alpha: int = 16) -> "LoRALinear":
        if linear.bias is not None:
            raise ValueError("LoRALinear wraps bias-free projections only")
        mod = cls(linear.in_features, linear.out_features, r, lora_alpha, device=linear.weight.device)
        with torch.no_grad():
            mod.weight.copy_(linear.weight.to(torch.bfloat16))
        return mod

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return lora_linear(x, self.weight, self.lora_A, self.lora_B, self.scaling)
