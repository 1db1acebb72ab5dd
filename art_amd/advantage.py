"""GRPO group-normalised advantages and the per-token broadcast / weights that
feed the loss kernels (host-side data preparation; vectorised).

Reference behaviour: src/art/local/tokenize.py:48-59 (advantage per trajectory,
population standard deviation, Python floats) and src/art/local/pack.py:97-100,
128-135 (per-token advantages and weights)."""
from __future__ import annotations

import numpy as np
import torch


def group_advantages(rewards, group_index) -> np.ndarray:
    """adv[i] = (r[i] - mean_g) / (std_g + 1e-6), float64, population std.

    rewards: float sequence [n]; group_index: int sequence [n] assigning each
    trajectory to a group (any integers).  Sums run in trajectory order, which
    is the order of the reference's Python ``sum``."""
    r = np.asarray(rewards, dtype=np.float64)
    g = np.asarray(group_index)
    if r.shape != g.shape or r.ndim != 1:
        raise ValueError("rewards and group_index must be 1-D and of equal length")
    if r.size == 0:
        return r.copy()
    _, inv = np.unique(g, return_inverse=True)
    n_groups = int(inv.max()) + 1
    count = np.bincount(inv, minlength=n_groups).astype(np.float64)
    mean = np.bincount(inv, weights=r, minlength=n_groups) / count
    dev = r - mean[inv]
    var = np.bincount(inv, weights=dev * dev, minlength=n_groups) / count
    std = np.sqrt(var)
    return dev / (std[inv] + 1e-6)


def keep_mask(advantages: np.ndarray) -> np.ndarray:
    """Trajectories the reference keeps: it skips advantage == 0 (tokenize.py:58-59)."""
    return np.asarray(advantages) != 0


def token_advantages(traj_id: torch.Tensor, advantages) -> torch.Tensor:
    """f32 [N,S]: advantage of each token's trajectory, 0 on padding (traj_id < 0)."""
    adv = torch.as_tensor(np.asarray(advantages, dtype=np.float64)).to(torch.float32).to(traj_id.device)
    safe = traj_id.clamp(min=0)
    return torch.where(traj_id >= 0, adv[safe], torch.zeros((), dtype=torch.float32, device=traj_id.device))


def token_weights(assistant_mask: torch.Tensor, traj_id: torch.Tensor) -> torch.Tensor:
    """f32 [N,S]: 1/(assistant tokens of the trajectory + 1e-6) on masked tokens,
    0 elsewhere, divided by the mean over masked tokens of the whole batch."""
    n_traj = int(traj_id.max().item()) + 1 if traj_id.numel() else 0
    valid = traj_id >= 0
    counts = torch.zeros(max(n_traj, 1), dtype=torch.float64, device=traj_id.device)
    counts.index_add_(0, traj_id[valid], assistant_mask[valid].to(torch.float64))
    per_traj = (1.0 / (counts + 1e-6)).to(torch.float32)
    w = torch.where(valid & assistant_mask, per_traj[traj_id.clamp(min=0)],
                    torch.zeros((), dtype=torch.float32, device=traj_id.device))
    sel = w[assistant_mask]
    if sel.numel():
        w = torch.where(assistant_mask, w / sel.mean(), w)
    return w
