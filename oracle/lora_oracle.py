"""CPU oracle of the LoRA linear.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference only configures this layer (src/art/local/state.py:86-92,
src/art/dev/model.py:52-67); the arithmetic lives in peft 0.15.2 / unsloth
2025.5.1, which are not in the reference tree.  PARITY UNPINNED against those
packages: no fixture of theirs exists to compare with.  This module states the
published formula y = base(x) + scaling * B(A(x)), scaling = alpha / r, and is
pinned by closed forms in tests/test_oracle_lora.py (explicit-loop evaluation
on tiny shapes, finite differences, the special cases B = 0 and A = 0)."""
from __future__ import annotations

import torch


def lora_linear(x, W, A, B, scale):
    """y = x W^T + scale * (x A^T) B^T."""
    return x @ W.t() + scale * ((x @ A.t()) @ B.t())


def lora_linear_grads(x_bf16, W_bf16, A, B, scale, g, dtype=torch.float32):
    """(y, dx, dA, dB) by autograd in `dtype` on up-casts of the inputs; W frozen."""
    x = x_bf16.to(dtype).clone().requires_grad_(True)
    A_ = A.to(dtype).clone().requires_grad_(True)
    B_ = B.to(dtype).clone().requires_grad_(True)
    y = lora_linear(x, W_bf16.to(dtype), A_, B_, scale)
    y.backward(g.to(dtype))
    return y.detach(), x.grad, A_.grad, B_.grad
