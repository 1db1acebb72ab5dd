"""Host-side mirror of the reference's loss module for the MI355X kernels.

Same callables, argument meaning and error behaviour as
``src/art/local/train.py`` of the reference, with the arithmetic done by the
artk HIP library:

=====================================  =========================================
reference (src/art/local/train.py)      here
=====================================  =========================================
``shift_tensor``            :284-285    ``shift_tensor`` (index op; the fused path
                                        never materialises shifted copies)
``_calculate_logprobs``     :245-281    ``_calculate_logprobs`` (autograd Function
                                        over artk_logprob_fwd / artk_logprob_bwd)
``calculate_logprobs``      :218-242    ``calculate_logprobs``
loss body of compute_loss   :111-151    ``grpo_loss`` (artk_grpo_loss) and
                                        ``fused_grpo_loss`` (artk_grpo_fused)
``get_compute_loss_fn``     :34-153     ``get_compute_loss_fn``
``train``                   :19-31      ``train`` (installs / restores the patches)
=====================================  =========================================
"""
from __future__ import annotations

import os
from contextlib import nullcontext
from typing import Callable, Optional

import torch

from . import ops


def shift_tensor(tensor: torch.Tensor, pad) -> torch.Tensor:
    """Position t gets element t+1 of its row; the last position gets ``pad``."""
    out = torch.empty_like(tensor)
    out[:, :-1] = tensor[:, 1:]
    out[:, -1] = pad
    return out


# -----------------------------------------------------------------------------
# logprobs
# -----------------------------------------------------------------------------
class _LogprobFn(torch.autograd.Function):
    """logprob[b, s] = log_softmax(hidden[b, s] @ lm_head.T)[ids[b, s]] without
    ever writing the [B*S, V] logits; the backward recomputes them chunk by chunk."""

    @staticmethod
    def forward(ctx, hidden, lm_head, ids, chunk_tokens):
        B, S, H = hidden.shape
        h2 = hidden.reshape(B * S, H)
        flat_ids = ids.reshape(B * S)
        logprob, lse = ops.logprob_fwd(h2, lm_head, flat_ids, False, S)
        ctx.save_for_backward(h2, lm_head, flat_ids, lse)
        ctx.shape = (B, S, H)
        ctx.chunk_tokens = chunk_tokens
        return logprob.view(B, S)

    @staticmethod
    def backward(ctx, grad_logprob):
        h2, lm_head, flat_ids, lse = ctx.saved_tensors
        B, S, H = ctx.shape
        g = grad_logprob.reshape(B * S).to(torch.float32).contiguous()
        d_hidden = ops.logprob_bwd(h2, lm_head, ops.transposed_weight(lm_head), flat_ids, False, S,
                                   lse, g, ctx.chunk_tokens)
        return d_hidden.view(B, S, H), None, None, None


def _as_vh(lm_head_t: torch.Tensor) -> torch.Tensor:
    """The bf16 [V, H] row-major weight behind the reference's ``lm_head_t`` ([H, V] view).
    When the view was made from the weight itself (``weight.t()``, as the reference does,
    src/art/local/train.py:76-78), the same tensor object comes back in every step, so the
    cached transposed copy of the weight is found again."""
    H, V = lm_head_t.shape
    base = lm_head_t._base
    if (base is not None and base.dim() == 2 and tuple(base.shape) == (V, H) and base.is_contiguous()
            and base.data_ptr() == lm_head_t.data_ptr() and lm_head_t.stride() == (1, H)):
        return ops.frozen_bf16(base)
    return lm_head_t.t().contiguous().to(torch.bfloat16)


def _calculate_logprobs(
    lm_head_t: torch.Tensor,  # [H, V]
    hidden_states: torch.Tensor,  # [B, S, H]
    next_input_ids: torch.Tensor,  # [B, S]
    chunk_size: int,
) -> torch.Tensor:  # [B, S] float32
    """Drop-in for the reference function of the same name.

    ``chunk_size`` keeps its contract (the sequence length must be divisible by
    it) but no longer bounds memory in the forward: no logits are stored at all.
    The result is float32 (the reference returns the hidden-state dtype)."""
    batch, seq_len, _ = hidden_states.shape
    assert (
        seq_len % chunk_size == 0
    ), f"Sequence length ({seq_len}) must be evenly divisible by chunk size ({chunk_size})"
    hidden = hidden_states.to(torch.bfloat16).contiguous()
    lm_head = _as_vh(lm_head_t)
    ids = next_input_ids.contiguous()
    return _LogprobFn.apply(hidden, lm_head, ids, ops.DEFAULT_CHUNK_TOKENS)


def calculate_logprobs(
    autocast_dtype: torch.dtype,
    trainer,
    input_ids: torch.Tensor,
    causal_mask: torch.Tensor,
    next_input_ids: torch.Tensor,
    lm_head_t: torch.Tensor,
    chunk_size: int,
    reference_logprobs: bool,
) -> torch.Tensor:
    """Model forward to hidden states, then ``_calculate_logprobs``.  With
    ``reference_logprobs`` the adapters are disabled and no graph is recorded."""
    model = trainer.model
    if reference_logprobs:
        unwrapped = trainer.accelerator.unwrap_model(model, keep_fp32_wrapper=False)
        adapters_off = unwrapped.disable_adapter()
        no_graph = torch.inference_mode()
    else:
        adapters_off = nullcontext()
        no_graph = nullcontext()
    with torch.autocast(device_type="cuda", dtype=autocast_dtype), no_graph, adapters_off:
        hidden_states = model(input_ids=input_ids, causal_mask=causal_mask).logits
    return _calculate_logprobs(lm_head_t, hidden_states, next_input_ids, chunk_size)


# -----------------------------------------------------------------------------
# loss
# -----------------------------------------------------------------------------
class _GRPOLossFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, new_logprobs, old, adv, mask, weights, ref, clip_lo, clip_hi, beta):
        B, S = new_logprobs.shape
        flat = lambda t: None if t is None else t.reshape(B * S).contiguous()
        scalars, coef = ops.grpo_loss(
            flat(new_logprobs.to(torch.float32)), flat(old), flat(adv), flat(mask), flat(weights),
            flat(ref), False, S, clip_lo, clip_hi, beta)
        ctx.save_for_backward(coef)
        ctx.shape = (B, S)
        ctx.in_dtype = new_logprobs.dtype
        ctx.mark_non_differentiable(scalars)
        return scalars[0], scalars

    @staticmethod
    def backward(ctx, g_loss, _g_scalars):
        (coef,) = ctx.saved_tensors
        g = (coef * g_loss).view(ctx.shape).to(ctx.in_dtype)
        return g, None, None, None, None, None, None, None, None


def grpo_loss(new_logprobs, old_logprobs, advantages, assistant_mask, weights, epsilon=0.2,
              epsilon_high=None, ref_logprobs=None, beta=0.0):
    """Clipped-surrogate loss on already shifted [B, S] tensors.

    Returns (loss, metrics) with metrics = {"policy_loss", "kl_div", "mask_count"}
    as 0-dim device tensors (no host sync)."""
    clip_lo, clip_hi = ops.clip_bounds(epsilon, epsilon_high)
    ref = ref_logprobs if beta > 0.0 else None
    loss, scalars = _GRPOLossFn.apply(
        new_logprobs, old_logprobs.to(torch.float32), advantages.to(torch.float32), assistant_mask,
        weights.to(torch.float32), None if ref is None else ref.to(torch.float32), clip_lo, clip_hi,
        float(beta))
    return loss, {"policy_loss": scalars[1], "kl_div": scalars[2], "mask_count": scalars[3]}


class _FusedGRPOLossFn(torch.autograd.Function):
    """loss(hidden) with d_hidden computed in the same pass (lm_head is frozen)."""

    @staticmethod
    def forward(ctx, hidden, lm_head, tokens, old, adv, mask, weights, ref, clip_lo, clip_hi, beta,
                chunk_tokens, skip_inactive):
        B, S, H = hidden.shape
        T = B * S
        flat = lambda t: None if t is None else t.reshape(T).contiguous()
        scalars, logprob, d_hidden = ops.grpo_fused(
            hidden.reshape(T, H), lm_head, ops.transposed_weight(lm_head), flat(tokens), flat(old),
            flat(adv), flat(mask), flat(weights), flat(ref), S, clip_lo, clip_hi, beta, chunk_tokens,
            skip_inactive=skip_inactive)
        ctx.save_for_backward(d_hidden)
        ctx.shape = (B, S, H)
        logprob = logprob.view(B, S)
        ctx.mark_non_differentiable(scalars, logprob)
        return scalars[0], scalars, logprob

    @staticmethod
    def backward(ctx, g_loss, _g_scalars, _g_logprob):
        (d_hidden,) = ctx.saved_tensors
        g = (d_hidden * g_loss).to(d_hidden.dtype).view(ctx.shape)
        return (g,) + (None,) * 12


def fused_grpo_loss(hidden_states, lm_head, tokens, logprobs, advantages, assistant_mask, weights,
                    epsilon=0.2, epsilon_high=None, ref_logprobs=None, beta=0.0,
                    chunk_tokens: int = ops.DEFAULT_CHUNK_TOKENS, skip_inactive: bool = False):
    """Loss of one packed batch from the model's hidden states, in one library call.

    Takes the *un-shifted* PackedTensors rows ([B, S]); equivalent to
    ``shift_tensor`` x5 + ``_calculate_logprobs`` + ``grpo_loss`` of the reference
    (src/art/local/train.py:76-151).  Returns (loss, metrics, new_logprobs).

    ``skip_inactive``: project only the positions whose loss term can be
    non-zero (the reference projects all of them and multiplies by the mask,
    train.py:145-151); loss, metrics and gradient are unchanged, new_logprobs is
    NaN at the skipped positions.

    metrics["dropped_rows"] counts positions whose sampled token has probability below
    e^-80 under the current policy: their gradient row is zero (see artk_grpo_fused).

    When no gradient can be asked for (``torch.no_grad()`` / ``inference_mode``, or hidden
    states that do not require grad) only the forward half runs: the lm_head projection
    without the stash of exponentials, then the loss kernels; no d_hidden GEMM.  Loss and
    logprobs are the same numbers; ``skip_inactive`` has no effect there."""
    clip_lo, clip_hi = ops.clip_bounds(epsilon, epsilon_high)
    ref = ref_logprobs if beta > 0.0 else None
    hidden = hidden_states.to(torch.bfloat16).contiguous()
    if not (torch.is_grad_enabled() and hidden_states.requires_grad):
        B, S, H = hidden.shape
        T = B * S
        flat = lambda t: None if t is None else t.reshape(T).contiguous()
        logprob, _ = ops.logprob_fwd(hidden.reshape(T, H), lm_head, flat(tokens), True, S)
        scalars, _ = ops.grpo_loss(
            logprob, flat(logprobs.to(torch.float32)), flat(advantages.to(torch.float32)),
            flat(assistant_mask), flat(weights.to(torch.float32)),
            None if ref is None else flat(ref.to(torch.float32)), True, S, clip_lo, clip_hi,
            float(beta), want_coef=False)
        metrics = {"policy_loss": scalars[1], "kl_div": scalars[2], "mask_count": scalars[3],
                   "dropped_rows": torch.zeros((), dtype=torch.float32, device=hidden.device)}
        return scalars[0], metrics, logprob.view(B, S)
    loss, scalars, logprob = _FusedGRPOLossFn.apply(
        hidden, lm_head, tokens, logprobs.to(torch.float32), advantages.to(torch.float32),
        assistant_mask, weights.to(torch.float32), None if ref is None else ref.to(torch.float32),
        clip_lo, clip_hi, float(beta), chunk_tokens, bool(skip_inactive))
    return loss, {"policy_loss": scalars[1], "kl_div": scalars[2], "mask_count": scalars[3],
                  "dropped_rows": scalars[4]}, logprob


def calculate_attn_bias(batch_size, seq_len, device, group_ids, parent_ids, autocast_dtype):
    """Additive block-causal bias [B, S, S]: position i sees j <= i of its own
    group or of its parent (reference: src/art/local/train.py:177-215)."""
    idx = torch.arange(seq_len, device=device)
    causal = (idx.unsqueeze(0) <= idx.unsqueeze(1)).unsqueeze(0)
    keys = group_ids.unsqueeze(1)
    visible = causal & ((group_ids.unsqueeze(2) == keys) | (parent_ids.unsqueeze(2) == keys))
    bias = torch.full((batch_size, seq_len, seq_len), float("-inf"), dtype=autocast_dtype, device=device)
    return bias.masked_fill_(visible, 0.0)


def get_compute_loss_fn(trainer) -> Callable[..., torch.Tensor]:
    """The ``compute_loss`` replacement that ``train`` installs on an HF/TRL trainer."""

    def compute_loss(model, inputs, return_outputs: bool = False, num_items_in_batch=None):
        config = inputs.pop("config")
        _config = inputs.pop("_config")

        optimizer = trainer.optimizer
        if optimizer:
            optimizer = getattr(optimizer, "optimizer", optimizer)
            for param_group in getattr(optimizer, "param_groups", None) or []:
                param_group["lr"] = config.learning_rate

        device = trainer.accelerator.device
        inputs = {key: tensor.to(device) for key, tensor in inputs.items()}

        mixed = os.environ.get("ACCELERATE_MIXED_PRECISION", "fp16")
        autocast_dtype = torch.float16 if mixed == "fp16" else torch.bfloat16
        if os.environ.get("UNSLOTH_FORCE_FLOAT32", "0") == "1":
            autocast_dtype = torch.float16

        batch_size, seq_len = inputs["tokens"].size()
        chunk_size = _config.get("logprob_calculation_chunk_size", 1024)
        assert (
            seq_len % chunk_size == 0
        ), f"Sequence length ({seq_len}) must be evenly divisible by chunk size ({chunk_size})"
        if _config.get("packed_attention_plans", False):
            # opt-in (no counterpart in the reference): the model's attention layers call
            # art_amd.attention.packed_attention and take, as `causal_mask`, one plan per packed row
            # made from the ids; the dense [B, S, S] bias (2 S^2 bytes per row) is never built
            attn_bias = [ops.attn_plan(inputs["group_ids"][b].contiguous(), inputs["parent_ids"][b].contiguous())
                         for b in range(batch_size)]
        else:
            attn_bias = calculate_attn_bias(batch_size, seq_len, device, inputs["group_ids"],
                                            inputs["parent_ids"], autocast_dtype)
        lm_head = trainer.model.get_output_embeddings().weight  # [V, H]
        if lm_head.requires_grad:
            # the fused step treats lm_head as frozen (LoRA on the attention / MLP projections only, the
            # reference's set-up): it computes no gradient for it, where the reference's autograd would
            raise NotImplementedError(
                "the output embedding is trainable (requires_grad=True, e.g. through modules_to_save): "
                "the fused GRPO step computes no gradient for lm_head; freeze it or use the reference loss")
        os.environ["UNSLOTH_RETURN_HIDDEN_STATES"] = "1"

        ref_logprobs = None
        if config.beta > 0.0:
            next_input_ids = shift_tensor(inputs["tokens"], 0)
            ref_logprobs = calculate_logprobs(autocast_dtype, trainer, inputs["tokens"], attn_bias,
                                              next_input_ids, lm_head.t(), chunk_size, True)
        with torch.autocast(device_type="cuda", dtype=autocast_dtype):
            hidden_states = trainer.model(input_ids=inputs["tokens"], causal_mask=attn_bias).logits
        del attn_bias

        epsilon = _config.get("epsilon", 0.2)
        epsilon_high = _config.get("epsilon_high", epsilon)
        loss, metrics, _ = fused_grpo_loss(
            hidden_states, ops.frozen_bf16(lm_head), inputs["tokens"], inputs["logprobs"],
            inputs["advantages"], inputs["assistant_mask"], inputs["weights"], epsilon, epsilon_high,
            ref_logprobs, config.beta, skip_inactive=True)  # new_logprobs are not used here

        # The reference appends `.item()` values here (train.py:147-150), one device
        # synchronisation per metric and step; the device scalars are kept instead and
        # converted when `log` averages them.
        trainer._metrics["learning_rate"].append(config.learning_rate)
        trainer._metrics["policy_loss"].append(metrics["policy_loss"].detach())
        if config.beta > 0.0:
            trainer._metrics["kl_div"].append(metrics["kl_div"].detach())
        # no counterpart in the reference: positions whose gradient row was dropped because the
        # sampled token has probability below e^-80 under the current policy (0 in a healthy run)
        trainer._metrics["dropped_rows"].append(metrics["dropped_rows"].detach())
        return loss

    return compute_loss


def get_log_fn(trainer, results_queue) -> Callable[..., None]:
    """Averages the per-step metrics and hands them to the service's queue
    (reference: src/art/local/train.py:156-174)."""

    def log(logs, start_time=None) -> None:
        metrics = {key: float(sum(vals) / len(vals)) for key, vals in trainer._metrics.items()}
        if next(iter(logs.keys())).startswith("eval_"):
            metrics = {f"eval_{key}": val for key, val in metrics.items()}
        merged = {**logs, **metrics}
        merged.pop("learning_rate", None)
        results_queue.put_nowait(merged)
        trainer._metrics.clear()

    return log


async def train(trainer, results_queue) -> None:
    """Run ``trainer.train()`` with the MI355X loss installed; always restore."""
    saved = (trainer.compute_loss, trainer.log)
    trainer.compute_loss = get_compute_loss_fn(trainer)
    trainer.log = get_log_fn(trainer, results_queue)
    try:
        trainer.train()
    finally:
        trainer.compute_loss, trainer.log = saved
