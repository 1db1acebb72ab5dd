"""MoE expert block with per-expert LoRA on the MI355X kernels.

Routing (top-k on the router logits, stable expert-contiguous permutation) and
the three per-expert projections (gate, up, down; each W_e x + scale B_e A_e x)
run in the artk library; the SiLU gating between them and the weighted
recombination of a token's k expert outputs are elementwise / gather steps done
with torch index ops in a fixed order.  The reference has no MoE code at this
commit; the shapes follow the Qwen3-30B-A3B-style benchmark configuration."""
from __future__ import annotations

import torch
from torch import nn

from . import ops


class _GroupedLoRAFn(torch.autograd.Function):
    """y_rows = per-expert LoRA linear of the sorted (token, expert) rows."""

    @staticmethod
    def forward(ctx, x, W, W_t, A, B, scale, routing, use_gather):
        gather = routing.row_token if use_gather else None
        A16 = A.detach().to(torch.bfloat16).contiguous()
        B16 = B.detach().to(torch.bfloat16).contiguous()
        y, xa = ops.moe_lora_grouped_fwd(x, gather, W, A16, B16, scale, routing)
        ctx.save_for_backward(x, W_t, A16, B16, xa)
        ctx.routing, ctx.scale, ctx.use_gather = routing, scale, use_gather
        ctx.dtypes = (A.dtype, B.dtype)
        return y

    @staticmethod
    def backward(ctx, g):
        x, W_t, A16, B16, xa = ctx.saved_tensors
        r = ctx.routing
        gather = r.row_token if ctx.use_gather else None
        dx_rows, dA, dB = ops.moe_lora_grouped_bwd(g.contiguous(), x, gather, W_t, A16, B16, xa,
                                                   ctx.scale, r)
        if ctx.use_gather:  # sum the k sorted rows of each token, slot order
            dx = dx_rows[r.inv_perm.long()].view(-1, r.k, dx_rows.shape[1]).float().sum(1).to(x.dtype)
        else:
            dx = dx_rows
        return dx, None, None, dA.to(ctx.dtypes[0]), dB.to(ctx.dtypes[1]), None, None, None


def grouped_lora_linear(x, W, W_t, A, B, scale, routing, use_gather: bool):
    return _GroupedLoRAFn.apply(x, W, W_t, A, B, float(scale), routing, use_gather)


def _fuse_adapters(A1, B1, A2, B2):
    """Adapters of two projections of the same input as one of rank r1 + r2:
    A stacked, B block-diagonal (autograd routes the gradients back to the four
    parameters; the off-diagonal blocks of dB belong to no adapter)."""
    A = torch.cat([A1, A2], 1)                                       # [E, r1 + r2, in]
    E, o1, r1 = B1.shape
    o2, r2 = B2.shape[1], B2.shape[2]
    top = torch.cat([B1, B1.new_zeros(E, o1, r2)], 2)
    bot = torch.cat([B2.new_zeros(E, o2, r1), B2], 2)
    return A, torch.cat([top, bot], 1)                               # [E, o1 + o2, r1 + r2]


class MoELoRAExperts(nn.Module):
    """E experts, each a gated MLP (gate/up [I,H], down [H,I]) with rank-r LoRA."""

    def __init__(self, hidden: int, intermediate: int, n_experts: int, top_k: int, r: int = 8,
                 lora_alpha: int = 16, device=None):
        super().__init__()
        self.top_k, self.scaling = top_k, lora_alpha / r
        bf = dict(device=device, dtype=torch.bfloat16)
        # gate and up read the same rows: they are stored as ONE [E, 2I, H] weight (gate rows first) so
        # that they run as one grouped product (one pass over x, twice the K length in the
        # input-gradient product); `gate_weight` / `up_weight` are views of it, not copies
        self.register_parameter("gate_up_weight", nn.Parameter(
            0.02 * torch.randn(n_experts, 2 * intermediate, hidden, **bf), requires_grad=False))
        self.register_parameter("down_weight", nn.Parameter(
            0.02 * torch.randn(n_experts, hidden, intermediate, **bf), requires_grad=False))
        shapes = {"gate": (intermediate, hidden), "up": (intermediate, hidden), "down": (hidden, intermediate)}
        for name, (o, i) in shapes.items():
            bound = 1.0 / i ** 0.5
            self.register_parameter(f"{name}_lora_A", nn.Parameter(
                (torch.rand(n_experts, r, i, device=device) * 2 - 1) * bound))
            self.register_parameter(f"{name}_lora_B", nn.Parameter(torch.zeros(n_experts, o, r, device=device)))
        self.intermediate = intermediate
        self._wt = {}

    @property
    def gate_weight(self) -> torch.Tensor:
        """[E, I, H] view of the gate rows of gate_up_weight."""
        return self.gate_up_weight[:, :self.intermediate]

    @property
    def up_weight(self) -> torch.Tensor:
        """[E, I, H] view of the up rows of gate_up_weight."""
        return self.gate_up_weight[:, self.intermediate:]

    def _transposed(self, name):
        w = getattr(self, f"{name}_weight")
        hit = self._wt.get(name)
        if hit is None or hit[0] != w._version or hit[1] != w.data_ptr():
            self._wt[name] = (w._version, w.data_ptr(), ops.transpose_batched(w))
        return self._wt[name][2]

    def _proj(self, name, x, routing, use_gather):
        return grouped_lora_linear(x, getattr(self, f"{name}_weight"), self._transposed(name),
                                   getattr(self, f"{name}_lora_A"), getattr(self, f"{name}_lora_B"),
                                   self.scaling, routing, use_gather)

    def forward(self, x: torch.Tensor, router_logits: torch.Tensor):
        """x bf16 [T,H], router_logits f32 [T,E] -> (y bf16 [T,H], routing)."""
        routing = ops.moe_route(router_logits.float().contiguous(), self.top_k)
        x = x.to(torch.bfloat16).contiguous()
        A_gu, B_gu = _fuse_adapters(self.gate_lora_A, self.gate_lora_B, self.up_lora_A, self.up_lora_B)
        gate_up = grouped_lora_linear(x, self.gate_up_weight, self._transposed("gate_up"), A_gu, B_gu,
                                      self.scaling, routing, True)
        gate, up = gate_up[:, :self.intermediate], gate_up[:, self.intermediate:]
        h = (torch.nn.functional.silu(gate.float()) * up.float()).to(torch.bfloat16)
        down = self._proj("down", h, routing, False)  # [T*k, H] in sorted order
        per_slot = down[routing.inv_perm.long()].view(x.shape[0], self.top_k, -1).float()
        y = (per_slot * routing.topk_w.unsqueeze(-1)).sum(1).to(torch.bfloat16)
        return y, routing
