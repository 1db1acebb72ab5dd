"""The committed GRPO fixture (tests/golden/grpo_small.npz: inputs as bit patterns, float64
evaluation of the reference's formulas as expected values) against the CPU oracle (here)
and against the kernels through the C-ABI (GPU)."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "oracle"))
import grpo_oracle  # noqa: E402

LP_TOL, LOSS_TOL, GRAD_TOL = 2e-3, 1e-3, 1e-2


def load():
    z = np.load(os.path.join(HERE, "golden", "grpo_small.npz"), allow_pickle=False)
    bf = lambda name: torch.from_numpy(z[name].copy()).view(torch.bfloat16)
    t = lambda name: torch.from_numpy(z[name].copy())
    return {
        "hidden": bf("hidden_bits"), "lm_head": bf("lm_head_bits"), "tokens": t("tokens"),
        "logprobs": t("logprobs"), "advantages": t("advantages"), "assistant_mask": t("assistant_mask"),
        "weights": t("weights"), "new": t("expect_new_logprobs"), "loss": float(z["expect_loss"]),
        "loss_scale": float(z["expect_loss_abs_terms"]), "mask_count": float(z["expect_mask_count"]),
        "d_hidden": t("expect_d_hidden"),
    }


def check(f, logprob, loss, mask_count, d_hidden):
    assert (logprob - f["new"]).abs().max().item() <= LP_TOL
    # the loss is a sum of terms of both signs: the tolerance is relative to the sum of their magnitudes
    assert abs(loss - f["loss"]) <= LOSS_TOL * f["loss_scale"]
    assert mask_count == f["mask_count"]
    rel = ((d_hidden.double() - f["d_hidden"].double()).norm() / f["d_hidden"].double().norm()).item()
    assert rel <= GRAD_TOL


def test_oracle_reproduces_fixture():
    f = load()
    ref = grpo_oracle.loss_and_grad(f["hidden"], f["lm_head"], f["tokens"], f["logprobs"], f["advantages"],
                                    f["assistant_mask"], f["weights"], chunk_size=64)
    mask_count = grpo_oracle.shift_tensor(f["assistant_mask"], False).sum().item()
    check(f, ref["logprobs"], ref["loss"].item(), mask_count, ref["d_hidden"])


@pytest.mark.gpu
def test_kernels_reproduce_fixture(artk_lib, gpu):
    from art_amd.train import fused_grpo_loss
    f = load()
    hidden = f["hidden"].to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(
        hidden, f["lm_head"].to(gpu), f["tokens"].to(gpu), f["logprobs"].to(gpu), f["advantages"].to(gpu),
        f["assistant_mask"].to(gpu), f["weights"].to(gpu))
    loss.backward()
    check(f, logprob.cpu(), loss.item(), metrics["mask_count"].item(), hidden.grad.float().cpu())
