"""Parity over shapes drawn at random (fixed seed, so the cases are the same in every
run): ragged token counts, odd tile counts, every supported rank, routing with empty and
single experts, id rows without any structure.  Same oracles and tolerances as the
per-operation tests."""
import os
import random
import sys

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "oracle"))
sys.path.insert(0, HERE)
import attn_oracle  # noqa: E402
import grpo_oracle  # noqa: E402
import lora_oracle  # noqa: E402
import moe_oracle  # noqa: E402

from art_amd import ops, synthetic  # noqa: E402
from art_amd.train import fused_grpo_loss  # noqa: E402

pytestmark = pytest.mark.gpu
TOL = 1e-2


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def draw(seed, n, fn):
    rng = random.Random(seed)
    return [fn(rng) for _ in range(n)]


LORA_CASES = draw(11, 10, lambda r: (r.randint(1, 1500), 64 * r.randint(1, 12), 64 * r.randint(1, 12),
                                     8 * r.randint(1, 8)))


@pytest.mark.parametrize("T,n_in,n_out,r", LORA_CASES)
def test_lora_random_shapes(artk_lib, gpu, T, n_in, n_out, r):
    print(f"sweep lora T={T} in={n_in} out={n_out} r={r}", flush=True)
    g = torch.Generator().manual_seed(T * 7 + r)
    bf = lambda *s, std=1.0: (std * torch.randn(*s, generator=g)).to(torch.bfloat16)
    x, W, A, B, up = bf(T, n_in), bf(n_out, n_in, std=0.02), bf(r, n_in, std=n_in ** -0.5), bf(n_out, r, std=0.02), bf(T, n_out)
    scale = 16.0 / r
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, scale, up)
    xd, Wd, Ad, Bd, upd = (t.to(gpu) for t in (x, W, A, B, up))
    y, xa = ops.lora_linear_fwd(xd, Wd, Ad, Bd, scale)
    dx, dA, dB = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL


def _moe_case(r):
    E = r.randint(1, 40)
    return (r.randint(1, 600), 64 * r.randint(1, 6), 64 * r.randint(1, 6), E, r.randint(1, min(E, 8)),
            8 * r.randint(1, 2), r.random() < 0.5)


MOE_CASES = draw(12, 10, _moe_case)


@pytest.mark.parametrize("T,H,I,E,k,r,use_gather", MOE_CASES)
def test_moe_random_shapes(artk_lib, gpu, T, H, I, E, k, r, use_gather):
    print(f"sweep moe T={T} H={H} I={I} E={E} k={k} r={r} gather={use_gather}", flush=True)
    g = torch.Generator().manual_seed(T + 31 * E)
    logits = torch.randn(T, E, generator=g)
    ref = moe_oracle.route(logits, k)
    rt = ops.moe_route(logits.to(gpu), k)
    assert torch.equal(rt.perm.cpu().long(), ref["perm"])
    assert torch.equal(rt.row_token.cpu().long(), ref["row_token"])
    assert torch.equal(rt.offsets.cpu().long(), ref["offsets"])
    n_rows = T * k
    x = torch.randn(T if use_gather else n_rows, H, generator=g).to(torch.bfloat16)
    W = (0.02 * torch.randn(E, I, H, generator=g)).to(torch.bfloat16)
    A = (H ** -0.5 * torch.randn(E, r, H, generator=g)).to(torch.bfloat16)
    B = (0.02 * torch.randn(E, I, r, generator=g)).to(torch.bfloat16)
    up = torch.randn(n_rows, I, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(x, ref["row_token"] if use_gather else None, W, A, B, 2.0,
                                                      ref["offsets"], up)
    gather = rt.row_token if use_gather else None
    y, xa = ops.moe_lora_grouped_fwd(x.to(gpu), gather, W.to(gpu), A.to(gpu), B.to(gpu), 2.0, rt)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), x.to(gpu), gather, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 2.0, rt)
    if use_gather:
        dx = dx[rt.inv_perm.long()].view(T, k, H).float().sum(1)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL


def _grpo_case(r):
    n_traj = r.choice([1, 2, 4, 8])
    L = r.randint(16, 300)
    T = n_traj * L
    return (T, 64 * r.randint(1, 6), 64 * r.randint(2, 200), n_traj, r.choice([0, r.randint(1, T)]),
            r.choice([0.0, 0.04]))


GRPO_CASES = draw(13, 10, _grpo_case)


@pytest.mark.parametrize("T,H,V,n_traj,chunk,beta", GRPO_CASES)
def test_grpo_random_shapes(artk_lib, gpu, T, H, V, n_traj, chunk, beta):
    print(f"sweep grpo T={T} H={H} V={V} traj={n_traj} chunk={chunk} beta={beta}", flush=True)
    case = synthetic.make_grpo_case("s", T + V, T, H, V, n_traj, min(4, n_traj), (0.2, 0.6))
    new = grpo_oracle.calculate_logprobs(case.lm_head.float().t(), case.hidden.float(),
                                         grpo_oracle.shift_tensor(case.tokens, 0), T)
    case.finish(new)
    g = torch.Generator().manual_seed(T)
    ref_lp = (new + 0.1 * torch.randn(1, T, generator=g)) if beta > 0 else None
    ref = grpo_oracle.loss_and_grad(case.hidden, case.lm_head, case.tokens, case.logprobs, case.advantages,
                                    case.assistant_mask, case.weights, chunk_size=T,
                                    **({"ref_logprobs": ref_lp, "beta": beta} if beta > 0 else {}))
    hidden = case.hidden.to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(
        hidden, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu), case.advantages.to(gpu),
        case.assistant_mask.to(gpu), case.weights.to(gpu), 0.2, 0.2,
        ref_lp.to(gpu) if ref_lp is not None else None, beta, chunk_tokens=chunk)
    loss.backward()
    assert (logprob.cpu() - ref["logprobs"]).abs().max().item() <= 2e-3
    # sums of terms of both signs: tolerance relative to the loss scale of a row (O(1e-2) here)
    assert abs(loss.item() - ref["loss"].item()) <= max(1e-3 * abs(ref["loss"].item()), 2e-5)
    assert rel_l2(hidden.grad.float().cpu(), ref["d_hidden"]) <= TOL


def _attn_case(r):
    hkv = r.choice([1, 2, 4])
    return (256 * r.randint(1, 8), hkv * r.choice([1, 2, 7]), hkv, r.choice([64, 128]),
            r.choice(["packed", "random_ids", "single"]))


ATTN_CASES = draw(14, 10, _attn_case)


@pytest.mark.parametrize("S,Hq,Hkv,D,kind", ATTN_CASES)
def test_attention_random_shapes(artk_lib, gpu, S, Hq, Hkv, D, kind):
    print(f"sweep attn S={S} Hq={Hq} Hkv={Hkv} D={D} ids={kind}", flush=True)
    g = torch.Generator().manual_seed(S + Hq)
    bf = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
    q, k, v, d_out = bf(S, Hq, D), bf(S, Hkv, D), bf(S, Hkv, D), bf(S, Hq, D)
    if kind == "packed":
        n_p = max(1, S // 700)
        group, parent = synthetic.packed_row_ids(S, S, n_p, 50, 3, (S // n_p - 60) // 3)
    elif kind == "random_ids":   # nothing contiguous: a handful of ids scattered over the row
        group = torch.randint(0, 6, (S,), generator=g, dtype=torch.int64)
        parent = torch.randint(0, 6, (S,), generator=g, dtype=torch.int64)
    else:                        # one sequence: plain causal attention
        group = torch.full((S,), 5, dtype=torch.int64)
        parent = group.clone()
    ref_out, ref_dq, ref_dk, ref_dv = attn_oracle.attention_grads(q, k, v, group, parent, d_out)
    plan = ops.attn_plan(group.to(gpu), parent.to(gpu))
    qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
    out, lse = ops.attn_fwd(qd, kd, vd, plan)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, out, lse, d_out.to(gpu), plan)
    assert rel_l2(out.float().cpu(), ref_out) <= TOL
    assert rel_l2(dq.float().cpu(), ref_dq) <= TOL
    assert rel_l2(dk.float().cpu(), ref_dk) <= TOL
    assert rel_l2(dv.float().cpu(), ref_dv) <= TOL
