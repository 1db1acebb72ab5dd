"""LoRA linear layer on the MI355X kernels.

``LoRALinear`` is the counterpart of the peft ``lora.Linear`` module that the
reference installs on the attention and MLP projections
(src/art/local/state.py:86-92; defaults r = 8, alpha = 16, no dropout,
``bias="none"``: src/art/dev/model.py:52-67).  The base weight is frozen, and so
is the base layer's own bias when it has one (Qwen2.5's q/k/v projections do;
peft keeps it and ``bias="none"`` means it is not trained); only ``lora_A`` and
``lora_B`` receive gradients."""
from __future__ import annotations

import math

import torch
from torch import nn

from . import ops


class _LoRALinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, lora_A, lora_B, scale, bias=None):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).to(torch.bfloat16).contiguous()
        A = lora_A.detach().to(torch.bfloat16).contiguous()
        B = lora_B.detach().to(torch.bfloat16).contiguous()
        y, xa = ops.lora_linear_fwd(x2, weight, A, B, scale, bias)
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
        return (dx.view(*ctx.lead, x2.shape[-1]).to(x_dtype), None, dA.to(a_dtype), dB.to(b_dtype), None, None)


class _LoRALinearNF4Fn(torch.autograd.Function):
    """The same linear with the frozen weight kept as NF4 codes (art_amd.quant.NF4Weight)."""

    @staticmethod
    def forward(ctx, x, w_nf4, lora_A, lora_B, scale, bias=None):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).to(torch.bfloat16).contiguous()
        A = lora_A.detach().to(torch.bfloat16).contiguous()
        B = lora_B.detach().to(torch.bfloat16).contiguous()
        y, xa = ops.lora_linear_fwd_nf4(x2, w_nf4, A, B, scale, bias)
        ctx.save_for_backward(x2, A, B, xa)
        ctx.w_nf4 = w_nf4
        ctx.scale = scale
        ctx.lead = lead
        ctx.param_dtypes = (lora_A.dtype, lora_B.dtype, x.dtype)
        return y.view(*lead, w_nf4.shape[0])

    @staticmethod
    def backward(ctx, g):
        x2, A, B, xa = ctx.saved_tensors
        g2 = g.reshape(-1, g.shape[-1]).to(torch.bfloat16).contiguous()
        dx, dA, dB = ops.lora_linear_bwd_nf4(g2, x2, ctx.w_nf4, A, B, xa, ctx.scale)
        a_dtype, b_dtype, x_dtype = ctx.param_dtypes
        return (dx.view(*ctx.lead, x2.shape[-1]).to(x_dtype), None, dA.to(a_dtype), dB.to(b_dtype), None, None)


def lora_linear(x, weight, lora_A, lora_B, scale: float, bias=None):
    """y = x W^T + bias + scale * (x A^T) B^T with gradients for x, A and B (W and bias frozen)."""
    if bias is not None:
        if bias.requires_grad:
            raise ValueError("the bias of a LoRA-wrapped linear is frozen (peft bias='none'); got requires_grad=True")
        bias = bias.detach().to(torch.bfloat16).contiguous()
    if not isinstance(weight, torch.Tensor):   # an NF4Weight
        return _LoRALinearNF4Fn.apply(x, weight, lora_A, lora_B, float(scale), bias)
    return _LoRALinearFn.apply(x, weight, lora_A, lora_B, float(scale), bias)


class LoRALinear(nn.Module):
    """Frozen bf16 linear with a trainable rank-r update; forward(x) -> y."""

    def __init__(self, in_features: int, out_features: int, r: int = 8, lora_alpha: int = 16,
                 device=None, dtype=torch.bfloat16, bias: bool = False):
        super().__init__()
        self.in_features, self.out_features, self.r = in_features, out_features, r
        self.scaling = lora_alpha / r
        self.weight = nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=torch.bfloat16),
                                   requires_grad=False)
        self.bias = (nn.Parameter(torch.zeros(out_features, device=device, dtype=torch.bfloat16), requires_grad=False)
                     if bias else None)
        self.lora_A = nn.Parameter(torch.empty(r, in_features, device=device, dtype=dtype))
        self.lora_B = nn.Parameter(torch.zeros(out_features, r, device=device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, std=0.02)
        nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))  # peft's default for A; B starts at zero
        nn.init.zeros_(self.lora_B)

    @classmethod
    def from_linear(cls, linear: nn.Linear, r: int = 8, lora_alpha: int = 16) -> "LoRALinear":
        mod = cls(linear.in_features, linear.out_features, r, lora_alpha, device=linear.weight.device,
                  bias=linear.bias is not None)
        with torch.no_grad():
            mod.weight.copy_(linear.weight.to(torch.bfloat16))
            if linear.bias is not None:
                mod.bias.copy_(linear.bias.to(torch.bfloat16))
        return mod

    @classmethod
    def from_nf4(cls, w_nf4, r: int = 8, lora_alpha: int = 16, bias=None) -> "LoRALinear":
        """Wrap a frozen weight that stays in its 4-bit storage form (art_amd.quant.NF4Weight): the
        module then holds no 16-bit copy of it, as with `load_in_4bit=True` in the reference
        (src/art/dev/model.py:29)."""
        n_out, n_in = w_nf4.shape
        dev = w_nf4.packed.device
        mod = cls.__new__(cls)
        nn.Module.__init__(mod)
        mod.in_features, mod.out_features, mod.r = n_in, n_out, r
        mod.scaling = lora_alpha / r
        mod.weight = None
        mod.weight_nf4 = w_nf4
        mod.bias = (nn.Parameter(bias.detach().to(torch.bfloat16).to(dev), requires_grad=False)
                    if bias is not None else None)
        mod.lora_A = nn.Parameter(torch.empty(r, n_in, device=dev, dtype=torch.bfloat16))
        mod.lora_B = nn.Parameter(torch.zeros(n_out, r, device=dev, dtype=torch.bfloat16))
        nn.init.kaiming_uniform_(mod.lora_A, a=math.sqrt(5))
        return mod

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        weight = self.weight if self.weight is not None else self.weight_nf4
        return lora_linear(x, weight, self.lora_A, self.lora_B, self.scaling, self.bias)


class _FusedLoRAFn(torch.autograd.Function):
    """Several projections of the same input through the library's multi-projection entry
    points: one launch walks the tiles of all of them over one x, the input gradient is one
    accumulation over all of them.  Weights, adapters, outputs and upstream gradients stay
    separate tensors: nothing is concatenated and no block-diagonal factor is built."""

    @staticmethod
    def forward(ctx, x, scale, n, *rest):
        weights, biases = rest[:n], rest[n:2 * n]
        As, Bs = rest[2 * n:3 * n], rest[3 * n:4 * n]
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).to(torch.bfloat16).contiguous()
        A16 = [a.detach().to(torch.bfloat16).contiguous() for a in As]
        B16 = [b.detach().to(torch.bfloat16).contiguous() for b in Bs]
        ys, xas = ops.lora_linear_multi_fwd(x2, list(weights), A16, B16, scale, list(biases))
        ctx.save_for_backward(x2, *weights, *A16, *B16, *xas)
        ctx.meta = (scale, n, lead, [a.dtype for a in As], [b.dtype for b in Bs], x.dtype)
        return tuple(y.view(*lead, y.shape[-1]) for y in ys)

    @staticmethod
    def backward(ctx, *gs):
        scale, n, lead, a_dt, b_dt, x_dt = ctx.meta
        saved = ctx.saved_tensors
        x2 = saved[0]
        weights, A16, B16, xas = (saved[1 + k * n:1 + (k + 1) * n] for k in range(4))
        g2 = []
        for g, w in zip(gs, weights):   # an output nobody used has no gradient: zeros
            g2.append(torch.zeros((x2.shape[0], w.shape[0]), dtype=torch.bfloat16, device=x2.device) if g is None
                      else g.reshape(-1, g.shape[-1]).to(torch.bfloat16).contiguous())
        dx, dAs, dBs = ops.lora_linear_multi_bwd(g2, x2, [ops.transposed_weight(w) for w in weights], list(A16),
                                                 list(B16), list(xas), scale)
        # gradients in the parameters' dtypes: one multi-tensor copy instead of a cast per tensor
        grads, want = list(dAs) + list(dBs), list(a_dt) + list(b_dt)
        cast = [i for i, (g_, t) in enumerate(zip(grads, want)) if g_.dtype != t]
        if cast:
            dst = [torch.empty_like(grads[i], dtype=want[i]) for i in cast]
            torch._foreach_copy_(dst, [grads[i] for i in cast])
            for i, d in zip(cast, dst):
                grads[i] = d
        return (dx.view(*lead, x2.shape[-1]).to(x_dt), None, None, *([None] * (2 * n)), *grads)


class FusedLoRALinear(nn.Module):
    """Projections that read the same activations (q/k/v, or gate/up) in one call each way:
    one persistent launch over the tiles of all of them (the narrow projections, k and v with
    256 or 512 columns, ride along with the wide one instead of leaving most of the GPU idle),
    one accumulation for the input gradient, one pass over x for all dA.  ``forward(x)``
    returns the tuple of the individual outputs.  The module holds the given layers and
    nothing else: no second copy of the frozen weights, no stacked adapters."""

    def __init__(self, layers):
        super().__init__()
        layers = list(layers)
        if len({l.in_features for l in layers}) != 1 or len({l.scaling for l in layers}) != 1:
            raise ValueError("fused projections need the same input size and scaling")
        if not 1 <= len(layers) <= 4:
            raise ValueError("one to four projections per call")
        if any(l.weight is None for l in layers):
            raise ValueError("fused projections need bf16 base weights (not NF4 codes)")
        self.outs = tuple(l.out_features for l in layers)
        self.ranks = tuple(l.r for l in layers)
        if sum(self.ranks) > 64:
            raise ValueError("sum of ranks above 64")
        self.scaling = layers[0].scaling
        self.layers = nn.ModuleList(layers)

    def forward(self, x: torch.Tensor):
        ls = self.layers
        for l in ls:
            if l.bias is not None and l.bias.requires_grad:
                raise ValueError("the bias of a LoRA-wrapped linear is frozen (peft bias='none')")
        biases = [None if l.bias is None else l.bias.detach().to(torch.bfloat16).contiguous() for l in ls]
        return _FusedLoRAFn.apply(x, float(self.scaling), len(ls), *[l.weight for l in ls], *biases,
                                  *[l.lora_A for l in ls], *[l.lora_B for l in ls])
