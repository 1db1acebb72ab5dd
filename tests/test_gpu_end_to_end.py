"""The pieces composed the way a training step uses them: one decoder layer
(LoRA projections + packed-row attention + gated MLP) feeding the fused GRPO
loss, backward through all of it, one fused AdamW step -- against the same
computation written with plain torch ops in fp32 on the CPU (dense bias from the
oracle, torch matmuls, torch.optim.AdamW)."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import attn_oracle  # noqa: E402
import grpo_oracle  # noqa: E402

from art_amd import synthetic  # noqa: E402
from art_amd.attention import attention_plans, packed_attention  # noqa: E402
from art_amd.lora import LoRALinear  # noqa: E402
from art_amd.optim import FlatParams, FusedAdamW  # noqa: E402
from art_amd.train import fused_grpo_loss  # noqa: E402

pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def rms(x):
    return x * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6).to(x.dtype)


def test_layer_loss_backward_step(artk_lib, gpu):
    torch.manual_seed(0)
    S, H, Hq, Hkv, D, I, V, r = 256, 128, 2, 1, 64, 256, 1024, 8
    case = synthetic.make_grpo_case("e2e", 5, S, H, V, 4, 4, 0.5)
    group, parent = synthetic.packed_row_ids(6, S, 1, 32, 4, 56)
    x0 = (0.5 * torch.randn(S, H)).to(torch.bfloat16)
    names = {"q": (H, Hq * D), "k": (H, Hkv * D), "v": (H, Hkv * D), "o": (Hq * D, H), "gate": (H, I),
             "up": (H, I), "down": (I, H)}
    # adapters live in one flat buffer; the modules' parameters are views of it
    shapes = {}
    for n, (i, o) in names.items():
        shapes[f"{n}.A"], shapes[f"{n}.B"] = (r, i), (o, r)
    flat = FlatParams(shapes, gpu)
    layers = {}
    for n, (i, o) in names.items():
        m = LoRALinear(i, o, r=r, lora_alpha=16, device=gpu, dtype=torch.float32)
        flat.param(f"{n}.A").copy_(m.lora_A.detach())
        flat.param(f"{n}.B").copy_(0.05 * torch.randn(o, r))
        m.lora_A = torch.nn.Parameter(flat.param(f"{n}.A"))
        m.lora_B = torch.nn.Parameter(flat.param(f"{n}.B"))
        m.lora_A.grad, m.lora_B.grad = flat.grad_of(f"{n}.A"), flat.grad_of(f"{n}.B")
        layers[n] = m
    master0 = flat.master.cpu().clone()

    def forward(x, lin, attn, loss_fn):
        hn = rms(x)
        q, k, v = lin("q", hn), lin("k", hn), lin("v", hn)
        ctx = attn(q.view(S, Hq, D), k.view(S, Hkv, D), v.view(S, Hkv, D)).reshape(S, Hq * D)
        x = x + lin("o", ctx)
        hn = rms(x)
        x = x + lin("down", torch.nn.functional.silu(lin("gate", hn)) * lin("up", hn))
        return loss_fn(rms(x))

    # ---- the same with torch ops, fp32, CPU
    P = {}
    for n in names:
        off_a, _ = flat.offsets[f"{n}.A"]
        P[n] = (layers[n].weight.detach().cpu().float(),
                master0[off_a:off_a + r * names[n][0]].view(r, names[n][0]).clone().requires_grad_(True),
                master0[flat.offsets[f"{n}.B"][0]:flat.offsets[f"{n}.B"][0] + names[n][1] * r]
                .view(names[n][1], r).clone().requires_grad_(True))

    def ref_attn(q, k, v):
        return attn_oracle.attention(q, k, v, group, parent)[0]

    def ref_loss(hid):
        new = grpo_oracle.calculate_logprobs(case.lm_head.float().t(), hid.view(1, S, H),
                                             grpo_oracle.shift_tensor(case.tokens, 0), S)
        sh = grpo_oracle.shift_tensor
        return grpo_oracle.grpo_loss(new, sh(case.logprobs, 0.0), sh(case.advantages, 0.0),
                                     sh(case.assistant_mask, False).float(), sh(case.weights, 0.0))[0]

    ref_lin = lambda n, t: t @ P[n][0].t() + 2.0 * (t @ P[n][1].t()) @ P[n][2].t()
    # old logprobs = the current policy's plus noise, as the synthetic cases define them
    with torch.no_grad():
        hid0 = forward(x0.float(), ref_lin, ref_attn, lambda hid: hid)
        case.finish(grpo_oracle.calculate_logprobs(case.lm_head.float().t(), hid0.view(1, S, H),
                                                   grpo_oracle.shift_tensor(case.tokens, 0), S))

    # ---- library path
    plans = attention_plans(group.to(gpu), parent.to(gpu))
    dev_case = case.to(gpu)
    loss = forward(
        x0.to(gpu), lambda n, t: layers[n](t), lambda q, k, v: packed_attention(q, k, v, plans),
        lambda hid: fused_grpo_loss(hid.view(1, S, H), dev_case.lm_head, dev_case.tokens, dev_case.logprobs,
                                    dev_case.advantages, dev_case.assistant_mask, dev_case.weights)[0])
    loss.backward()
    grads = flat.grad.cpu().clone()
    opt = FusedAdamW(flat, lr=1e-3)
    opt.step()

    ref = forward(x0.float(), ref_lin, ref_attn, ref_loss)
    ref.backward()
    # the loss is a small difference of O(1) per-token terms (ratios near 1, advantages of both signs):
    # compare on that scale, the chain runs in bf16 on the GPU
    assert abs(loss.item() - ref.item()) <= 5e-4
    for n in names:
        for which, idx in (("A", 1), ("B", 2)):
            off, shape = flat.offsets[f"{n}.{which}"]
            got = grads[off:off + P[n][idx].numel()].view(shape)
            assert rel_l2(got, P[n][idx].grad) <= 5e-2, (n, which)
    # the optimizer moved every adapter against its (clipped) gradient
    moved = flat.master.cpu() - master0 * (1 - 1e-3 * 0.1)
    nz = grads != 0
    assert torch.all(torch.sign(moved[nz]) == -torch.sign(grads[nz]))
