"""`get_compute_loss_fn` (the patch installed on the trainer,
src/art/local/train.py:34-153) driven with a stand-in trainer whose model is an
embedding table: loss, KL branch with disabled adapters, learning-rate
override, metric store, gradient w.r.t. the model -- against the oracle."""
import collections
import os
import sys
import types
from contextlib import contextmanager

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import grpo_oracle  # noqa: E402

from art_amd import ops, synthetic  # noqa: E402
from art_amd.train import get_compute_loss_fn  # noqa: E402

pytestmark = pytest.mark.gpu


class TinyModel(torch.nn.Module):
    """hidden = emb[token] + adapter[token]; `disable_adapter()` drops the second term."""

    def __init__(self, V, H, lm_head, dev):
        super().__init__()
        self.emb = torch.nn.Parameter(torch.randn(V, H, device=dev) * 0.5)
        self.adapter = torch.nn.Parameter(torch.randn(V, H, device=dev) * 0.05)
        self.head = torch.nn.Linear(H, V, bias=False, device=dev, dtype=torch.bfloat16)
        with torch.no_grad():
            self.head.weight.copy_(lm_head)
        self.head.weight.requires_grad_(False)
        self.use_adapter = True

    def get_output_embeddings(self):
        return self.head

    @contextmanager
    def disable_adapter(self):
        self.use_adapter = False
        try:
            yield
        finally:
            self.use_adapter = True

    def forward(self, input_ids, causal_mask):
        self.last_mask = causal_mask
        h = self.emb[input_ids]
        if self.use_adapter:
            h = h + self.adapter[input_ids]
        return types.SimpleNamespace(logits=h)


@pytest.mark.parametrize("beta", [0.0, 0.05])
def test_compute_loss_patch(artk_lib, gpu, beta):
    S, H, V = 512, 128, 4096
    case = synthetic.make_grpo_case("cl", 7, S, H, V, 4, 4, 0.5)
    torch.manual_seed(1)
    model = TinyModel(V, H, case.lm_head.to(gpu), gpu)
    group, parent = synthetic.packed_row_ids(8, S, 1, 64, 4, 112)
    # old logprobs from the current policy (+ noise), as the synthetic cases define them
    with torch.no_grad():
        hid = (model.emb + model.adapter)[case.tokens[0].to(gpu)].to(torch.bfloat16).cpu()
        ref_hid = model.emb[case.tokens[0].to(gpu)].to(torch.bfloat16).cpu()
    nxt = grpo_oracle.shift_tensor(case.tokens, 0)
    case.finish(grpo_oracle.calculate_logprobs(case.lm_head.float().t(), hid.float().view(1, S, H), nxt, S))

    opt = types.SimpleNamespace(param_groups=[{"lr": 1.0}])
    trainer = types.SimpleNamespace(
        model=model, optimizer=types.SimpleNamespace(optimizer=opt),
        accelerator=types.SimpleNamespace(device=gpu, unwrap_model=lambda m, keep_fp32_wrapper=False: m),
        _metrics=collections.defaultdict(list))
    os.environ["ACCELERATE_MIXED_PRECISION"] = "bf16"
    compute_loss = get_compute_loss_fn(trainer)
    inputs = {"tokens": case.tokens, "group_ids": group.view(1, S), "parent_ids": parent.view(1, S),
              "input_pos": torch.arange(S).view(1, S), "assistant_mask": case.assistant_mask,
              "logprobs": case.logprobs, "advantages": case.advantages, "weights": case.weights,
              "config": types.SimpleNamespace(learning_rate=3e-6, beta=beta),
              "_config": {"logprob_calculation_chunk_size": 256, "epsilon": 0.2}}
    inputs_backup = {k: v for k, v in inputs.items() if k not in ("config", "_config")}
    loss = compute_loss(model, inputs)
    loss.backward()

    ref_lp = None
    if beta > 0:
        ref_lp = grpo_oracle.calculate_logprobs(case.lm_head.float().t(), ref_hid.float().view(1, S, H), nxt, S)
    want = grpo_oracle.loss_and_grad(hid.view(1, S, H), case.lm_head, case.tokens, case.logprobs, case.advantages,
                                     case.assistant_mask, case.weights, chunk_size=S, ref_logprobs=ref_lp,
                                     beta=beta)
    assert abs(loss.item() - want["loss"].item()) <= 1e-3 * abs(want["loss"].item()) + 2e-6
    assert opt.param_groups[0]["lr"] == 3e-6
    assert len(trainer._metrics["policy_loss"]) == 1 and trainer._metrics["learning_rate"] == [3e-6]
    assert (len(trainer._metrics["kl_div"]) == 1) == (beta > 0)
    if beta > 0:
        assert abs(float(trainer._metrics["kl_div"][0]) - want["kl"].item()) <= 2e-3 * abs(want["kl"].item()) + 1e-7
    # gradient reaches the model: rows of the embedding table touched by active positions
    g = torch.zeros(V, H)
    g.index_add_(0, case.tokens[0], want["d_hidden"][0].float())
    got = model.adapter.grad.cpu()
    assert ((got - g).norm() / g.norm()).item() <= 2e-2
    # chunk size must divide the row length, as in the reference
    bad = dict(inputs, config=inputs_config(beta), _config={"logprob_calculation_chunk_size": 300})
    with pytest.raises(AssertionError):
        compute_loss(model, bad)
    # the dense bias by default; with the opt-in the model gets one attention plan per row instead
    assert torch.is_tensor(model.last_mask) and model.last_mask.shape == (1, S, S)
    again = {k: v for k, v in inputs_backup.items()}
    again["config"] = inputs_config(beta)
    again["_config"] = {"logprob_calculation_chunk_size": 256, "epsilon": 0.2, "packed_attention_plans": True}
    loss2 = compute_loss(model, again)
    assert isinstance(model.last_mask, list) and len(model.last_mask) == 1
    assert isinstance(model.last_mask[0], ops.AttnPlan) and model.last_mask[0].S == S
    assert loss2.item() == loss.item()
    # a trainable output embedding is refused: the fused step computes no gradient for it
    model.head.weight.requires_grad_(True)
    try:
        with pytest.raises(NotImplementedError, match="lm_head"):
            compute_loss(model, dict(inputs_backup, config=inputs_config(beta),
                                     _config={"logprob_calculation_chunk_size": 256}))
    finally:
        model.head.weight.requires_grad_(False)


def inputs_config(beta):
    return types.SimpleNamespace(learning_rate=3e-6, beta=beta)
