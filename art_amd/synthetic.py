"""Deterministic synthetic workloads of the benchmark configurations.

All random draws happen on the CPU from ``torch.Generator().manual_seed(seed)``
in a fixed order (hidden, lm_head, tokens, mask fractions, rewards, noise) so
the host checker and the device see identical bits."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Optional

import numpy as np
import torch

from .advantage import group_advantages, token_advantages, token_weights


@dataclass
class GRPOCase:
    name: str
    hidden: torch.Tensor          # bf16 [1,S,H]
    lm_head: torch.Tensor         # bf16 [V,H]
    tokens: torch.Tensor          # int64 [1,S]
    assistant_mask: torch.Tensor  # bool [1,S]
    advantages: torch.Tensor      # f32 [1,S]
    weights: torch.Tensor         # f32 [1,S]
    logprobs: Optional[torch.Tensor]  # f32 [1,S] old logprobs (NaN off-mask); filled by finish()
    traj_id: torch.Tensor         # int64 [1,S]
    group_of_traj: np.ndarray     # int64 [n_traj]
    rewards: np.ndarray           # float64 [n_traj]
    traj_advantages: np.ndarray   # float64 [n_traj]
    noise: torch.Tensor           # f32 [1,S]
    epsilon: float = 0.2
    beta: float = 0.0
    extra: dict = field(default_factory=dict)

    def finish(self, new_logprobs: torch.Tensor) -> "GRPOCase":
        """old[t+1] = new[t] + noise[t]; NaN wherever the token is not an assistant token."""
        new = new_logprobs.detach().to("cpu", torch.float32).view(1, -1)
        old = torch.full_like(new, float("nan"))
        old[:, 1:] = new[:, :-1] + self.noise[:, :-1]
        old = torch.where(self.assistant_mask, old, torch.full_like(old, float("nan")))
        self.logprobs = old
        return self

    def to(self, device) -> "GRPOCase":
        moved = {}
        for k, v in self.__dict__.items():
            moved[k] = v.to(device) if isinstance(v, torch.Tensor) else v
        return GRPOCase(**moved)


def span_mask(length: int, n_assistant: int) -> torch.Tensor:
    """4 gaps and 4 assistant spans alternating, gap first; the first three spans
    are equal and the last takes the remainder; gaps likewise with the remainder
    going to the first gap."""
    n_assistant = max(0, min(n_assistant, length - 4))
    spans = [n_assistant // 4] * 3
    spans.append(n_assistant - sum(spans))
    gap_total = length - n_assistant
    gaps = [gap_total // 4] * 4
    gaps[0] += gap_total - sum(gaps)
    pieces = []
    for g, s in zip(gaps, spans):
        pieces.append(torch.zeros(g, dtype=torch.bool))
        pieces.append(torch.ones(s, dtype=torch.bool))
    return torch.cat(pieces)


def make_grpo_case(name: str, seed: int, T: int, H: int, V: int, n_traj: int, group_size: int,
                   mask_frac, rewards: str = "uniform", noise_std: float = 0.05) -> GRPOCase:
    """``mask_frac``: a float (same density for every trajectory) or a (lo, span)
    pair for per-trajectory densities lo + span * U[0,1).  ``rewards``: "uniform"
    (U[0,1)) or "bernoulli" (p = 0.5: zero-variance groups give zero advantage)."""
    assert T % n_traj == 0 and n_traj % group_size == 0
    L = T // n_traj
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16).view(1, T, H)
    lm_head = (0.02 * torch.randn(V, H, generator=g)).to(torch.bfloat16)
    tokens = torch.randint(0, V, (1, T), generator=g, dtype=torch.int64)
    if isinstance(mask_frac, tuple):
        fr = mask_frac[0] + mask_frac[1] * torch.rand(n_traj, generator=g)
    else:
        fr = torch.full((n_traj,), float(mask_frac))
    if rewards == "uniform":
        r = torch.rand(n_traj, generator=g, dtype=torch.float64).numpy()
    elif rewards == "bernoulli":
        r = (torch.rand(n_traj, generator=g) < 0.5).to(torch.float64).numpy()
    else:
        raise ValueError(rewards)
    noise = noise_std * torch.randn(1, T, generator=g)

    mask = torch.cat([span_mask(L, int(round(float(f) * L))) for f in fr]).view(1, T)
    traj_id = torch.arange(n_traj, dtype=torch.int64).repeat_interleave(L).view(1, T)
    group_of_traj = np.arange(n_traj, dtype=np.int64) // group_size
    adv = group_advantages(r, group_of_traj)
    return GRPOCase(
        name=name, hidden=hidden, lm_head=lm_head, tokens=tokens, assistant_mask=mask,
        advantages=token_advantages(traj_id, adv), weights=token_weights(mask, traj_id),
        logprobs=None, traj_id=traj_id, group_of_traj=group_of_traj, rewards=r,
        traj_advantages=adv, noise=noise)


# The benchmark configurations.
def config1() -> GRPOCase:
    """Qwen2.5-0.5B shape: 4 trajectories of 512 tokens, one group of 4, ~50 % mask."""
    return make_grpo_case("C1-qwen2.5-0.5b", 1001, 2048, 896, 151936, 4, 4, 0.5)


def config3() -> GRPOCase:
    """Qwen2.5-7B shape: 32 trajectories of 512 tokens in 8 groups of 4, 40 % mask."""
    return make_grpo_case("C3-qwen2.5-7b", 1003, 16384, 3584, 152064, 32, 4, 0.4)


def config4() -> GRPOCase:
    """Qwen2.5-14B shape: 16 trajectories of 2048 tokens in 4 groups of 4,
    20-70 % mask per trajectory, Bernoulli rewards."""
    return make_grpo_case("C4-qwen2.5-14b", 1004, 32768, 5120, 152064, 16, 4, (0.2, 0.5),
                          rewards="bernoulli")


def packed_row_ids(seed: int, S: int, n_prompts: int, prompt_len: int, n_completions: int,
                   completion_len: int):
    """group_ids / parent_ids (int64 [S]) of one packed row the way the packer lays
    it out (reference: src/art/local/pack.py:84-93, 139-140): each prompt's tokens
    carry group = parent = prompt id; each of its completions gets a fresh random
    64-bit group id and parent = prompt id; the tail of the row is padding (-1, -1)."""
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(-(2 ** 62), 2 ** 62, (n_prompts * (1 + n_completions),), generator=g)
    group, parent = [], []
    k = 0
    for _ in range(n_prompts):
        pid = int(ids[k]); k += 1
        group += [pid] * prompt_len
        parent += [pid] * prompt_len
        for _ in range(n_completions):
            cid = int(ids[k]); k += 1
            group += [cid] * completion_len
            parent += [pid] * completion_len
    assert len(group) <= S, "row too short for the requested layout"
    pad = S - len(group)
    group += [-1] * pad
    parent += [-1] * pad
    return torch.tensor(group, dtype=torch.int64), torch.tensor(parent, dtype=torch.int64)
