"""Pins of the CPU oracle (oracle/grpo_oracle.py).  The reference ships no tests
or golden vectors for this path, so each function is checked against what the
mathematics fixes: closed forms, library routines, hand-computed known answers,
brute force and finite differences, chosen so that a dropped term, a wrong sign
or an off-by-one index fails."""
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import grpo_oracle as O  # noqa: E402


# ---- shift_tensor ------------------------------------------------------------
def test_shift_closed_form():
    t = torch.arange(12).view(2, 6)
    out = O.shift_tensor(t, -7)
    for b in range(2):
        for s in range(6):
            assert out[b, s].item() == (t[b, s + 1].item() if s + 1 < 6 else -7)
    m = torch.tensor([[True, False, True]])
    assert O.shift_tensor(m, False).tolist() == [[False, True, False]]
    f = torch.tensor([[1.5, float("nan"), 2.5]])
    o = O.shift_tensor(f, 0.0)
    assert math.isnan(o[0, 0].item()) and o[0, 1].item() == 2.5 and o[0, 2].item() == 0.0
    assert o.dtype == f.dtype and O.shift_tensor(t, 0).dtype == torch.int64


# ---- calculate_logprobs -------------------------------------------------------
def test_logprobs_equal_log_softmax_fp64():
    g = torch.Generator().manual_seed(0)
    B, S, H, V = 2, 12, 16, 50
    h = torch.randn(B, S, H, generator=g, dtype=torch.float64)
    W = torch.randn(V, H, generator=g, dtype=torch.float64)
    ids = torch.randint(0, V, (B, S), generator=g)
    want = torch.log_softmax(h @ W.t(), -1).gather(-1, ids.unsqueeze(-1)).squeeze(-1)
    for chunk in (1, 3, 4, 12):
        got = O.calculate_logprobs(W.t(), h, ids, chunk)
        assert torch.allclose(got, want, atol=1e-12), chunk
    # the V logprobs of one position are a distribution
    all_ids = torch.arange(V).view(1, V)
    lp = O.calculate_logprobs(W.t(), h[:1, :1].expand(1, V, H).contiguous(), all_ids, V)
    assert abs(lp.exp().sum().item() - 1.0) < 1e-12


def test_logprobs_brute_force_tiny():
    h = torch.tensor([[[1.0, 2.0]]], dtype=torch.float64)
    W = torch.tensor([[0.5, -1.0], [2.0, 0.0], [0.0, 1.0]], dtype=torch.float64)
    logits = [0.5 - 2.0, 2.0, 2.0]
    lse = math.log(sum(math.exp(z) for z in logits))
    for y in range(3):
        got = O.calculate_logprobs(W.t(), h, torch.tensor([[y]]), 1).item()
        assert abs(got - (logits[y] - lse)) < 1e-14


def test_logprobs_dtype_follows_hidden_and_chunk_assert():
    h = torch.randn(1, 4, 8).to(torch.bfloat16)
    W = torch.randn(10, 8)
    out = O.calculate_logprobs(W.t(), h, torch.zeros(1, 4, dtype=torch.int64), 2)
    assert out.dtype == torch.bfloat16
    with pytest.raises(AssertionError):
        O.calculate_logprobs(W.t(), h, torch.zeros(1, 4, dtype=torch.int64), 3)


# ---- grpo_loss -----------------------------------------------------------------
def test_loss_ratio_clip_known_answers():
    """r = [1, 1.1, 1.3, 0.7, 1.2, 0.8], A = [2, 2, 2, 2, -1, -1], eps = 0.2:
    -min(rA, clip(r)A) = [-2, -2.2, -2.4, -1.4, 1.2, 0.8] and its derivative with
    respect to r is [-2, -2, 0, -2, 1, 1] (clip passes the gradient on its bounds,
    min takes the unclipped branch when it is smaller)."""
    r = torch.tensor([[1.0, 1.1, 1.3, 0.7, 1.2, 0.8]], dtype=torch.float64)
    A = torch.tensor([[2.0, 2.0, 2.0, 2.0, -1.0, -1.0]], dtype=torch.float64)
    new = r.log().clone().requires_grad_(True)
    old = torch.zeros_like(new)
    ones = torch.ones_like(new)
    loss, mpl, mkl = O.grpo_loss(new, old, A, ones, ones, 0.2)
    want = [-2.0, -2.2, -2.4, -1.4, 1.2, 0.8]
    assert abs(mpl.item() - sum(want) / (6 + 1e-6)) < 1e-12
    assert mkl.item() == 0.0 and loss.item() == mpl.item()
    loss.backward()
    d_dr = [-2.0, -2.0, 0.0, -2.0, 1.0, 1.0]
    for i in range(6):  # d/dnew = r * d/dr, divided by the mask count
        assert abs(new.grad[0, i].item() - r[0, i].item() * d_dr[i] / (6 + 1e-6)) < 1e-12


def test_loss_asymmetric_clip():
    new = torch.tensor([[math.log(1.25)]], dtype=torch.float64)
    one = torch.ones(1, 1, dtype=torch.float64)
    # eps_high = 0.3: 1.25 is inside the range -> -r A ; eps_high = 0.2 -> clipped at 1.2
    l1, _, _ = O.grpo_loss(new, torch.zeros_like(new), one, one, one, 0.2, 0.3)
    l2, _, _ = O.grpo_loss(new, torch.zeros_like(new), one, one, one, 0.2, None)
    assert abs(l1.item() * (1 + 1e-6) + 1.25) < 1e-12
    assert abs(l2.item() * (1 + 1e-6) + 1.2) < 1e-12


def test_loss_special_cases():
    g = torch.Generator().manual_seed(1)
    S = 16
    new = -torch.rand(1, S, generator=g, dtype=torch.float64) * 3
    adv = torch.randn(1, S, generator=g, dtype=torch.float64)
    w = torch.rand(1, S, generator=g, dtype=torch.float64)
    m = (torch.rand(1, S, generator=g) < 0.5).to(torch.float64)
    # old == new: ratio 1, loss = -sum(A w m) / (sum m + 1e-6)
    loss, _, _ = O.grpo_loss(new, new.clone(), adv, m, w)
    assert abs(loss.item() + (adv * w * m).sum().item() / (m.sum().item() + 1e-6)) < 1e-12
    # NaN old behaves like old == new
    loss_nan, _, _ = O.grpo_loss(new, torch.full_like(new, float("nan")), adv, m, w)
    assert loss_nan.item() == loss.item()
    # zero advantage: zero loss and zero gradient
    n2 = new.clone().requires_grad_(True)
    l0, _, _ = O.grpo_loss(n2, new + 0.1, torch.zeros_like(adv), m, w)
    l0.backward()
    assert l0.item() == 0.0 and n2.grad.abs().max().item() == 0.0
    # empty mask: denominator 1e-6, numerator 0
    le, _, _ = O.grpo_loss(new, new + 0.1, adv, torch.zeros_like(m), w)
    assert le.item() == 0.0


def test_loss_kl_term_closed_form():
    new = torch.tensor([[-1.0, -2.0]], dtype=torch.float64)
    ref = torch.tensor([[-1.5, -1.0]], dtype=torch.float64)
    one = torch.ones_like(new)
    loss, mpl, mkl = O.grpo_loss(new, new.clone(), torch.zeros_like(new), one, one, ref_logprobs=ref, beta=0.5)
    d = [-0.5, 1.0]
    want = sum(math.exp(x) - x - 1 for x in d) / (2 + 1e-6)
    assert abs(mkl.item() - want) < 1e-12 and abs(loss.item() - 0.5 * want) < 1e-12 and mpl.item() == 0.0


# ---- compute_loss / d_hidden -----------------------------------------------------
def _tiny_case(dtype=torch.float64):
    g = torch.Generator().manual_seed(3)
    S, H, V = 8, 6, 11
    h = torch.randn(1, S, H, generator=g).to(torch.bfloat16)
    W = (0.3 * torch.randn(V, H, generator=g)).to(torch.bfloat16)
    tokens = torch.randint(0, V, (1, S), generator=g)
    mask = torch.tensor([[False, True, True, False, True, True, True, False]])
    old = torch.full((1, S), float("nan"))
    old[mask] = -2.0 + 0.3 * torch.randn(int(mask.sum()), generator=g)
    adv = torch.randn(1, S, generator=g)
    w = torch.rand(1, S, generator=g) + 0.5
    return h, W, tokens, old, adv, mask, w


def test_dhidden_closed_form_and_finite_differences():
    h, W, tokens, old, adv, mask, w = _tiny_case()
    out = O.loss_and_grad(h, W, tokens, old, adv, mask, w, chunk_size=4, dtype=torch.float64)
    # closed form: d_hidden[t] = c_t (W[y_t] - softmax_t W), c_t from the loss kernel formula
    h64, W64 = h.double()[0], W.double()
    y = O.shift_tensor(tokens, 0)[0]
    p = torch.softmax(h64 @ W64.t(), -1)
    new = out["logprobs"][0]
    o = O.shift_tensor(old.double(), 0.0)[0]
    o = torch.where(torch.isnan(o), new, o)
    a = O.shift_tensor(adv.double(), 0.0)[0]
    m = O.shift_tensor(mask, False)[0].double()
    ww = O.shift_tensor(w.double(), 0.0)[0]
    ratio = (new - o).exp()
    inside = (ratio >= 0.8) & (ratio <= 1.2)
    take = inside | (ratio * a < ratio.clamp(0.8, 1.2) * a)
    c = torch.where(take, -ratio * a, torch.zeros_like(a)) * ww * m / (m.sum() + 1e-6)
    want = c.unsqueeze(1) * (W64[y] - p @ W64)
    assert torch.allclose(out["d_hidden"][0], want, atol=1e-12)
    # finite differences on a few coordinates
    def f(hh):
        return O.compute_loss(hh, W.double(), tokens, old.double(), adv.double(), mask, w.double(), chunk_size=4)[0].item()
    base = h.double()
    for (s, k) in [(1, 0), (4, 3), (6, 5)]:
        e = torch.zeros_like(base)
        e[0, s, k] = 1e-6
        fd = (f(base + e) - f(base - e)) / 2e-6
        assert abs(fd - out["d_hidden"][0, s, k].item()) < 1e-7


def test_last_position_and_unmasked_rows_have_no_gradient():
    h, W, tokens, old, adv, mask, w = _tiny_case()
    out = O.loss_and_grad(h, W, tokens, old, adv, mask, w, chunk_size=8, dtype=torch.float64)
    m = O.shift_tensor(mask, False)[0]
    assert out["d_hidden"][0][~m].abs().max().item() == 0.0
    assert not m[-1]  # the pad at the end of the row


# ---- advantages / weights ----------------------------------------------------------
def test_advantages_known_answers():
    adv = O.grpo_advantages([[1.0, 0.0, 0.0, 1.0], [0.5, 0.5, 0.5, 0.5], [3.0], []])
    # mean 0.5, population std 0.5
    v = 0.5 / (0.5 + 1e-6)
    assert adv[0] == [v, -v, -v, v]
    assert adv[1] == [0.0, 0.0, 0.0, 0.0] and adv[2] == [0.0] and adv[3] == []
    a = O.grpo_advantages([[2.0, 4.0, 4.0, 6.0]])[0]  # mean 4, std sqrt(2)
    s = math.sqrt(2.0) + 1e-6
    assert a == [-2 / s, 0.0, 0.0, 2 / s]


def test_token_weights_invariants():
    mask = torch.tensor([[True, True, False, True, False, False, True, False]])
    traj = torch.tensor([[0, 0, 0, 1, 1, 1, 2, -1]])
    w = O.token_weights(mask, traj)
    assert w[~mask].abs().max().item() == 0.0
    assert abs(w[mask].mean().item() - 1.0) < 1e-6
    # trajectory 0 has 2 assistant tokens, 1 and 2 have one: weights 1/2 : 1 : 1 before normalisation
    assert abs(w[0, 0].item() / w[0, 3].item() - 0.5) < 1e-5 and abs(w[0, 3].item() - w[0, 6].item()) < 1e-6
