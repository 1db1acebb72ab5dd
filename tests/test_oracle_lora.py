"""Pins of oracle/lora_oracle.py: explicit-loop evaluation on tiny shapes, finite
differences, and the special cases B = 0 and A = 0."""
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import lora_oracle as L  # noqa: E402


def _tiny():
    g = torch.Generator().manual_seed(0)
    T, n_in, n_out, r = 3, 4, 5, 2
    x = torch.randn(T, n_in, generator=g, dtype=torch.float64)
    W = torch.randn(n_out, n_in, generator=g, dtype=torch.float64)
    A = torch.randn(r, n_in, generator=g, dtype=torch.float64)
    B = torch.randn(n_out, r, generator=g, dtype=torch.float64)
    up = torch.randn(T, n_out, generator=g, dtype=torch.float64)
    return x, W, A, B, up


def test_forward_explicit_loops():
    x, W, A, B, _ = _tiny()
    s = 2.0
    y = L.lora_linear(x, W, A, B, s)
    for t in range(3):
        for o in range(5):
            base = sum(W[o, i].item() * x[t, i].item() for i in range(4))
            low = sum(B[o, k].item() * sum(A[k, i].item() * x[t, i].item() for i in range(4)) for k in range(2))
            assert abs(y[t, o].item() - (base + s * low)) < 1e-12


def test_gradients_closed_form_and_finite_differences():
    x, W, A, B, up = _tiny()
    s = 2.0
    y, dx, dA, dB = L.lora_linear_grads(x, W, A, B, s, up, dtype=torch.float64)
    assert torch.allclose(dx, up @ W + s * (up @ B) @ A, atol=1e-12)
    assert torch.allclose(dA, s * (up @ B).t() @ x, atol=1e-12)
    assert torch.allclose(dB, s * up.t() @ (x @ A.t()), atol=1e-12)
    f = lambda xx, AA, BB: (L.lora_linear(xx, W, AA, BB, s) * up).sum().item()
    e = 1e-6
    d = torch.zeros_like(A); d[1, 2] = e
    assert abs((f(x, A + d, B) - f(x, A - d, B)) / (2 * e) - dA[1, 2].item()) < 1e-6
    d = torch.zeros_like(B); d[3, 0] = e
    assert abs((f(x, A, B + d) - f(x, A, B - d)) / (2 * e) - dB[3, 0].item()) < 1e-6
    d = torch.zeros_like(x); d[2, 1] = e
    assert abs((f(x + d, A, B) - f(x - d, A, B)) / (2 * e) - dx[2, 1].item()) < 1e-6


def test_zero_factors():
    x, W, A, B, up = _tiny()
    y, dx, dA, dB = L.lora_linear_grads(x, W, A, torch.zeros_like(B), 2.0, up, dtype=torch.float64)
    assert torch.equal(y, x @ W.t()) and dA.abs().max().item() == 0.0
    y, dx, dA, dB = L.lora_linear_grads(x, W, torch.zeros_like(A), B, 2.0, up, dtype=torch.float64)
    assert dB.abs().max().item() == 0.0
