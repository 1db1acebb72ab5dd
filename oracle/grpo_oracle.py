"""CPU oracle of the GRPO hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain torch on the CPU, the algorithm of the reference
for the per-token logprob / loss path.  Only ``tests/``, ``__graft_entry__.smoke``
and the ``cpu_baseline`` leg of ``bench.py`` may import it; nothing under
``art_amd/`` does.  It is the checker, never the product.

Each function cites the reference lines it follows (paths relative to the
reference tree).  The functions are dtype-generic like the reference: fed fp32
up-casts of bf16 inputs they give the fp32 evaluation that the parity tests
compare against; fed bf16 they reproduce the reference's production dtype.

How each function is pinned (the reference ships no tests or golden vectors):
  shift_tensor            closed form out[t] = in[t+1]; brute force on tiny arrays
  calculate_logprobs      equals log_softmax(h @ W.T)[y] (library routine, fp64);
                          chunk-size invariance; sum_v exp(logprob_v) == 1
  grpo_loss               hand-computed known answers for ratio / clip / min
                          gradients; special cases old == new, adv == 0, NaN old
  grpo_advantages         hand-computed groups; zero-variance group -> zeros
  token_weights           invariant mean(weights[mask]) == 1, weights[~mask] == 0
  d_hidden (autograd)     closed form c_t (W[y_t] - softmax_t W); finite differences
These checks live in tests/test_oracle_*.py.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch


def shift_tensor(tensor: torch.Tensor, pad) -> torch.Tensor:
    """out[:, t] = in[:, t+1], out[:, -1] = pad.  Follows src/art/local/train.py:284-285."""
    out = torch.full_like(tensor, pad)
    out[:, :-1] = tensor[:, 1:]
    return out


def calculate_logprobs(
    lm_head_t: torch.Tensor,  # [H, V]
    hidden_states: torch.Tensor,  # [B, S, H]
    next_input_ids: torch.Tensor,  # [B, S]
    chunk_size: int,
) -> torch.Tensor:
    """Chunked matmul -> gather -> logsumexp -> subtract.

    Follows src/art/local/train.py:245-281: output allocated in the dtype of the
    hidden states (:253-257), lm_head cast to it (:259), S/chunk chunks (:262).
    """
    batch, seq_len, _ = hidden_states.shape
    assert seq_len % chunk_size == 0  # train.py:82-84
    out = torch.empty((batch, seq_len), dtype=hidden_states.dtype, device=hidden_states.device)
    lm_head_t = lm_head_t.to(hidden_states.dtype)
    for i in range(0, seq_len, chunk_size):
        logits = torch.matmul(hidden_states[:, i : i + chunk_size, :], lm_head_t)
        ids = next_input_ids[:, i : i + chunk_size]
        selected = torch.gather(logits, -1, ids.unsqueeze(-1)).squeeze(-1)
        out[:, i : i + chunk_size] = selected - torch.logsumexp(logits, dim=-1)
    return out


def grpo_loss(
    new_logprobs: torch.Tensor,  # [B, S] position frame
    old_logprobs: torch.Tensor,  # [B, S] already shifted; NaN = missing
    advantages: torch.Tensor,  # [B, S] already shifted
    assistant_mask: torch.Tensor,  # [B, S] already shifted, same dtype as new_logprobs
    weights: torch.Tensor,  # [B, S] already shifted
    epsilon: float = 0.2,
    epsilon_high: Optional[float] = None,
    ref_logprobs: Optional[torch.Tensor] = None,
    beta: float = 0.0,
):
    """Clipped-surrogate GRPO loss.  Follows src/art/local/train.py:119-151.

    Returns (loss, mean_policy_loss, mean_kl).
    """
    old_logprobs = torch.where(torch.isnan(old_logprobs), new_logprobs.detach(), old_logprobs)
    prob_ratio = torch.exp(new_logprobs - old_logprobs)
    if epsilon_high is None:
        epsilon_high = epsilon
    policy_loss = -torch.min(
        prob_ratio * advantages,
        torch.clip(prob_ratio, 1 - epsilon, 1 + epsilon_high) * advantages,
    )
    if ref_logprobs is not None:
        diff = ref_logprobs - new_logprobs
        kl_div = torch.exp(diff) - diff - 1.0
    else:
        kl_div = torch.zeros_like(policy_loss)
    policy_loss = policy_loss * weights * assistant_mask
    kl_div = kl_div * weights * assistant_mask
    denom = assistant_mask.sum() + 1e-6
    mean_policy_loss = policy_loss.sum() / denom
    mean_kl = kl_div.sum() / denom
    return mean_policy_loss + beta * mean_kl, mean_policy_loss, mean_kl


def compute_loss(
    hidden_states: torch.Tensor,  # [B, S, H]
    lm_head: torch.Tensor,  # [V, H]
    tokens: torch.Tensor,  # [B, S] int64, un-shifted
    logprobs: torch.Tensor,  # [B, S] f32, un-shifted, NaN = missing
    advantages: torch.Tensor,  # [B, S] f32, un-shifted
    assistant_mask: torch.Tensor,  # [B, S] bool, un-shifted
    weights: torch.Tensor,  # [B, S] f32, un-shifted
    epsilon: float = 0.2,
    epsilon_high: Optional[float] = None,
    chunk_size: int = 1024,
    ref_logprobs: Optional[torch.Tensor] = None,
    beta: float = 0.0,
):
    """The loss part of compute_loss, src/art/local/train.py:76-151, given the
    hidden states that the model forward would have produced (:239-241).

    Returns (loss, mean_policy_loss, mean_kl, new_logprobs).
    """
    lm_head_t = lm_head.t()  # train.py:76-78
    next_input_ids = shift_tensor(tokens, 0)  # :79
    new_logprobs = calculate_logprobs(lm_head_t, hidden_states, next_input_ids, chunk_size)
    old = shift_tensor(logprobs, 0.0)  # :112
    adv = shift_tensor(advantages, 0.0)  # :113
    mask = shift_tensor(assistant_mask, False).to(new_logprobs.dtype)  # :114-116
    w = shift_tensor(weights, 0.0)  # :117
    loss, mpl, mkl = grpo_loss(new_logprobs, old, adv, mask, w, epsilon, epsilon_high, ref_logprobs, beta)
    return loss, mpl, mkl, new_logprobs


def loss_and_grad(hidden_bf16, lm_head_bf16, tokens, logprobs, advantages, assistant_mask, weights,
                  epsilon=0.2, epsilon_high=None, chunk_size=1024, ref_logprobs=None, beta=0.0,
                  dtype=torch.float32):
    """fp32 (or fp64) evaluation on the exactly representable up-casts of the bf16
    inputs, with autograd for d_hidden (lm_head frozen: src/art/dev/model.py:54-62).

    Returns dict(loss, policy_loss, kl, logprobs, d_hidden)."""
    h = hidden_bf16.to(dtype).clone().requires_grad_(True)
    w = lm_head_bf16.to(dtype)
    ref = None if ref_logprobs is None else ref_logprobs.to(dtype)
    loss, mpl, mkl, new = compute_loss(
        h, w, tokens, logprobs.to(dtype), advantages.to(dtype), assistant_mask, weights.to(dtype),
        epsilon, epsilon_high, chunk_size, ref, beta,
    )
    loss.backward()
    return {
        "loss": loss.detach(),
        "policy_loss": mpl.detach(),
        "kl": mkl.detach(),
        "logprobs": new.detach(),
        "d_hidden": h.grad.detach(),
    }


def grpo_advantages(rewards_by_group: Sequence[Sequence[float]]) -> list[list[float]]:
    """Per group: (r - mean) / (population std + 1e-6) in Python floats.

    Follows src/art/local/tokenize.py:48-57.  (The reference then drops
    trajectories whose advantage is exactly 0, :58-59; callers decide.)"""
    out = []
    for group in rewards_by_group:
        n = len(group)
        if n == 0:
            out.append([])
            continue
        mean = sum(group) / n
        std = math.sqrt(sum((r - mean) ** 2 for r in group) / n)
        out.append([(r - mean) / (std + 1e-6) for r in group])
    return out


def token_weights(assistant_mask: torch.Tensor, traj_id: torch.Tensor) -> torch.Tensor:
    """Per-token weights of one packed batch.  Follows src/art/local/pack.py:98-100
    (1 / (assistant tokens of the trajectory + 1e-6) on every token of it) and
    :128-135 (zero off-mask, divide by the mean over masked tokens).

    assistant_mask: bool [N, S]; traj_id: int64 [N, S], -1 on padding."""
    mask_flat = assistant_mask.reshape(-1)
    ids_flat = traj_id.reshape(-1)
    values = [0.0] * mask_flat.numel()
    counts: dict[int, int] = {}
    for m, i in zip(mask_flat.tolist(), ids_flat.tolist()):
        if i >= 0:
            counts[i] = counts.get(i, 0) + int(m)
    for k, i in enumerate(ids_flat.tolist()):
        if i >= 0:
            values[k] = 1 / (counts[i] + 1e-6)
    w = torch.tensor(values).reshape(assistant_mask.shape)  # float32, like torch.tensor(list)
    w = torch.where(assistant_mask, w, torch.zeros_like(w))
    w[assistant_mask] /= w[assistant_mask].mean()
    return w
