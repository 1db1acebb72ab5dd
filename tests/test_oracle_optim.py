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


# ---- 8-bit block-wise moments -------------------------------------------------------------
def code_books():
    from art_amd.optim import dynamic_code_book
    return dynamic_code_book(True).numpy(), dynamic_code_book(False).numpy()


def test_code_books_shape_and_quantiser_fixed_points():
    import numpy as np

    b1, b2 = code_books()
    for b, lo in ((b1, -1.0), (b2, 0.0)):
        assert b.shape == (256,) and np.all(np.diff(b) >= 0) and b[-1] == 1.0 and b.min() >= lo
        assert 0.0 in b
        # every distinct entry quantises to itself (to the last of equal entries)
        idx = optim_oracle.nearest_code(b, b)
        assert np.array_equal(b[idx], b)
        # a value between two entries goes to the nearer one
        u = np.unique(b)
        mid = (u[:-1] + u[1:]) / 2
        lower = optim_oracle.nearest_code(b, (mid - (u[1:] - u[:-1]) * 0.25).astype(np.float32))
        upper = optim_oracle.nearest_code(b, (mid + (u[1:] - u[:-1]) * 0.25).astype(np.float32))
        assert np.array_equal(b[lower], u[:-1]) and np.array_equal(b[upper], u[1:])
    assert b1.min() < -0.99 and (b2 >= 0).all()
    # resolution near 1 (where a block's largest element sits): better than 1 %
    assert np.diff(np.unique(b1))[-8:].max() < 0.02 and np.diff(np.unique(b2))[-8:].max() < 0.01


def test_8bit_first_step_is_the_closed_form_up_to_the_code_book():
    import numpy as np

    b1, b2 = code_books()
    rng = np.random.default_rng(0)
    n = 512
    p0 = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 0.1).astype(np.float32)
    z8, za = np.zeros(n, np.uint8), np.zeros(2, np.float32)
    lr, wd, eps, betas = 1e-2, 0.1, 1e-8, (0.9, 0.99)
    p, c1, c2, a1, a2 = optim_oracle.adamw8bit_step(p0, g, z8, z8, za, za, b1, b2, lr, betas, eps, wd, 1)
    # step 1 from zero state: bias-corrected m / sqrt(v) = sign(g); decay multiplies after the update
    want = (p0 - lr * g / (np.abs(g) + eps)) * (1 - lr * wd)
    assert np.allclose(p, want, rtol=2e-5, atol=1e-7)
    # stored moments: block maxima exact, elements within the local step of the book
    m, v = 0.1 * g, 0.01 * g * g
    assert np.allclose(a1, np.abs(m).reshape(2, 256).max(1), rtol=1e-6)
    assert np.allclose(a2, v.reshape(2, 256).max(1), rtol=1e-6)
    dm = b1[c1] * np.repeat(a1, 256)
    dv = b2[c2] * np.repeat(a2, 256)
    assert np.abs(dm - m).max() <= 0.05 * np.abs(m).max()
    assert np.abs(dv - v).max() <= 0.05 * v.max()
    big = np.abs(m) > 0.2 * np.abs(m).max()
    assert (np.abs(dm - m)[big] / np.abs(m)[big]).max() < 0.06


def test_8bit_tracks_fp32_adamw():
    """60 steps on the same gradients: parameters stay close to torch.optim.AdamW's (the moments
    carry a few per cent of quantisation error each, the parameter path averages it out)."""
    import numpy as np

    b1, b2 = code_books()
    gen = torch.Generator().manual_seed(1)
    n = 1024
    p0 = torch.randn(n, generator=gen) * 0.05
    base = torch.randn(n, generator=gen)
    grads = [(base + 0.5 * torch.randn(n, generator=gen)) * 0.01 for _ in range(60)]
    lr, wd, eps, betas = 1e-3, 0.1, 1e-8, (0.9, 0.99)
    ref_p, _, _, _ = optim_oracle.adamw_steps(p0, grads, lr, betas, eps, wd, 0.0)
    p = p0.numpy().copy()
    c1 = c2 = np.zeros(n, np.uint8)
    a1 = a2 = np.zeros(n // 256, np.float32)
    for t, g in enumerate(grads, 1):
        p, c1, c2, a1, a2 = optim_oracle.adamw8bit_step(p, g.numpy(), c1, c2, a1, a2, b1, b2, lr, betas, eps, wd, t)
    moved = (ref_p - p0).abs().mean().item()
    err = np.abs(p - ref_p.numpy()).mean()
    assert moved > 0.02 and err < 0.05 * moved
