"""Flat storage and fused AdamW for the adapter parameters (fp32 or 8-bit block-wise moments).

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


def dynamic_code_book(signed: bool, max_exponent_bits: int = 7, total_bits: int = 8) -> torch.Tensor:
    """The 256-entry "dynamic" code book of the 8-bit block-wise optimizers (Dettmers et al.,
    "8-bit Optimizers via Block-wise Quantization", 2022, section 2.2 / appendix: a sign bit,
    a run of exponent bits that selects a power of ten, and a linear fraction with the
    remaining bits), ascending, in [-1, 1] (signed: exp_avg) or [0, 1] (unsigned: exp_avg_sq).
    Restated from the published construction; bitsandbytes itself is not available here, so
    the book is an explicit input of the kernel and a checkpoint's own book can be passed instead."""
    data = []
    non_sign_bits = total_bits - 1
    additional_items = 2 ** (non_sign_bits - max_exponent_bits) - 1
    for i in range(max_exponent_bits):
        if signed:
            fraction_items = int(2 ** (i + non_sign_bits - max_exponent_bits) + 1)
        else:
            fraction_items = int(2 ** (i + non_sign_bits - max_exponent_bits + 1) + 1)
        boundaries = torch.linspace(0.1, 1, fraction_items, dtype=torch.float64)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        scale = 10.0 ** (-(max_exponent_bits - 1) + i)
        data += (scale * means).tolist()
        if signed:
            data += (-scale * means).tolist()
    if additional_items > 0:
        boundaries = torch.linspace(0.1, 1, additional_items + 1, dtype=torch.float64)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        scale = 10.0 ** (-(max_exponent_bits - 1) + max_exponent_bits - 1)
        data += (scale * means).tolist()
        if signed:
            data += (-scale * means).tolist()
    data += [0.0, 1.0]
    data += [0.0] * (2 ** total_bits - len(data))
    return torch.tensor(sorted(data), dtype=torch.float32)


class FusedAdamW8bit:
    """FusedAdamW with the moments kept the way the reference's `paged_adamw_8bit` keeps them
    (src/art/dev/model.py:75): one byte per element and moment plus one fp32 maximum per block of
    256 elements, 2 bytes of optimizer state per parameter instead of 8."""

    def __init__(self, flat: FlatParams, lr: float = 5e-6, betas=(0.9, 0.99), eps: float = 1e-8,
                 weight_decay: float = 0.1, max_grad_norm: float = 0.1):
        self.flat = flat
        self.lr, self.betas, self.eps = lr, betas, eps
        self.weight_decay, self.max_grad_norm = weight_decay, max_grad_norm
        dev = flat.master.device
        n, nb = flat.numel, (flat.numel + 255) // 256
        self.state1 = torch.zeros(n, dtype=torch.uint8, device=dev)
        self.state2 = torch.zeros(n, dtype=torch.uint8, device=dev)
        self.absmax1 = torch.zeros(nb, dtype=torch.float32, device=dev)
        self.absmax2 = torch.zeros(nb, dtype=torch.float32, device=dev)
        self.qmap1 = dynamic_code_book(True).to(dev)
        self.qmap2 = dynamic_code_book(False).to(dev)
        self.steps = 0

    def step(self) -> torch.Tensor:
        """One update; returns the squared gradient norm before clipping (device scalar)."""
        self.steps += 1
        f = self.flat
        sumsq = ops.sumsq(f.grad)
        clip = self.max_grad_norm is not None and self.max_grad_norm > 0
        ops.adamw8bit_step(f.master, f.grad, self.state1, self.state2, self.absmax1, self.absmax2, self.qmap1,
                           self.qmap2, f.shadow, self.lr, self.betas[0], self.betas[1], self.eps,
                           self.weight_decay, self.steps, sumsq if clip else None,
                           self.max_grad_norm if clip else 0.0)
        return sumsq

    def exp_avg(self) -> torch.Tensor:
        """The first moment, dequantised (for inspection and tests)."""
        return self.qmap1[self.state1.long()] * self.absmax1.repeat_interleave(256)[: self.flat.numel]

    def exp_avg_sq(self) -> torch.Tensor:
        return self.qmap2[self.state2.long()] * self.absmax2.repeat_interleave(256)[: self.flat.numel]
