"""Flat storage and fused AdamW for the adapter parameters.

The reference lets HF Trainer step `paged_adamw_8bit` over ~400 small LoRA
tensors and clip their global gradient norm at 0.1 (src/art/dev/model.py:69-85).
`FlatParams` places all of them in one fp32 buffer (gradients, moments and the
bf16 copy that the GEMM kernels read likewise), so `FusedAdamW.step()` is one
norm and one update launch over contiguous memory.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Sequence, Tuple

import torch

from . import ops


class FlatParams:
    """fp32 master copy, gradient and bf16 shadow of a set of tensors as views into
    three flat buffers.  Each tensor starts on a 16-byte boundary."""

    def __init__(self, shapes: Dict[str, Sequence[int]], device: torch.device):
        self.offsets: Dict[str, Tuple[int, Tuple[int, ...]]] = {}
        n = 0
        for name, shape in shapes.items():
            numel = 1
            for d in shape:
                numel *= d
            self.offsets[name] = (n, tuple(shape))
            n += (numel + 7) // 8 * 8
        self.numel = n
        self.master = torch.zeros(n, dtype=torch.float32, device=device)
        self.grad = torch.zeros(n, dtype=torch.float32, device=device)
        self.shadow = torch.zeros(n, dtype=torch.bfloat16, device=device)

    def _view(self, buf: torch.Tensor, name: str) -> torch.Tensor:
        off, shape = self.offsets[name]
        numel = 1
        for d in shape:
            numel *= d
        return buf[off:off + numel].view(shape)

    def param(self, name: str) -> torch.Tensor:
        return self._view(self.master, name)

    def grad_of(self, name: str) -> torch.Tensor:
        return self._view(self.grad, name)

    def bf16(self, name: str) -> torch.Tensor:
        return self._view(self.shadow, name)

    def sync_shadow(self) -> None:
        self.shadow.copy_(self.master)

    def zero_grad(self) -> None:
        self.grad.zero_()


class FusedAdamW:
    """AdamW with decoupled weight decay (torch.optim.AdamW's rule) and global
    gradient-norm clipping (torch.nn.utils.clip_grad_norm_'s rule) on a FlatParams.
    Defaults are the reference's trainer settings."""

    def __init__(self, flat: FlatParams, lr: float = 5e-6, betas=(0.9, 0.99), eps: float = 1e-8,
                 weight_decay: float = 0.1, max_grad_norm: float = 0.1):
        self.flat = flat
        self.lr, self.betas, self.eps = lr, betas, eps
        self.weight_decay, self.max_grad_norm = weight_decay, max_grad_norm
        self.exp_avg = torch.zeros_like(flat.master)
        self.exp_avg_sq = torch.zeros_like(flat.master)
        self.steps = 0

    def step(self) -> torch.Tensor:
        """One update; returns the squared gradient norm before clipping (device scalar)."""
        self.steps += 1
        f = self.flat
        sumsq = ops.sumsq(f.grad)
        clip = self.max_grad_norm is not None and self.max_grad_norm > 0
        ops.adamw_step(f.master, f.grad, self.exp_avg, self.exp_avg_sq, f.shadow, self.lr, self.betas[0],
                       self.betas[1], self.eps, self.weight_decay, self.steps,
                       sumsq if clip else None, self.max_grad_norm if clip else 0.0)
        return sumsq
