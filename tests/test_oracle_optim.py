"""Pins of the optimizer oracle (torch.optim.AdamW + clip_grad_norm_): closed form
of the first step and of the clip coefficient.  CPU only."""
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import optim_oracle  # noqa: E402


def test_first_step_closed_form():
    p0 = torch.tensor([1.0, -2.0, 0.5, 3.0], dtype=torch.float64)
    g = torch.tensor([0.3, -0.1, 0.0, 2.0], dtype=torch.float64)
    lr, wd, eps = 1e-2, 0.1, 1e-8
    p, m, v, norms = optim_oracle.adamw_steps(p0, [g], lr, (0.9, 0.99), eps, wd, 0.0)
    # bias-corrected moments of step 1 are g and g^2
    want = p0 * (1 - lr * wd) - lr * g / (g.abs() + eps)
    assert torch.allclose(p.double(), want, rtol=1e-6, atol=1e-9)
    assert torch.allclose(m.double(), 0.1 * g, rtol=1e-6) and torch.allclose(v.double(), 0.01 * g * g, rtol=1e-6)
    assert abs(norms[0] - float((g * g).sum())) < 1e-6


def test_clip_coefficient():
    p0 = torch.zeros(3)
    g = torch.tensor([3.0, 4.0, 0.0])          # norm 5
    lr = 1.0
    p, m, v, norms = optim_oracle.adamw_steps(p0, [g], lr, (0.0, 0.0), 0.0, 0.0, 0.1)
    assert abs(norms[0] - 25.0) < 1e-4
    # clipped gradient = g * 0.1 / (5 + 1e-6); with betas 0 and eps 0 the step is lr * sign(g)
    assert torch.allclose(p[:2], torch.tensor([-1.0, -1.0]))
    assert torch.allclose(m, g * (0.1 / (5 + 1e-6)), rtol=1e-6)
