"""GPU parity of the MoE expert path: routing and permutation bit-exact, grouped
per-expert LoRA projections within rel-L2 1e-2 of the fp32 oracle."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import moe_oracle  # noqa: E402

from art_amd import ops  # noqa: E402
from art_amd.moe import MoELoRAExperts  # noqa: E402

pytestmark = pytest.mark.gpu
TOL = 1e-2


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def check_routing(logits, k, gpu):
    ref = moe_oracle.route(logits, k)
    r = ops.moe_route(logits.to(gpu), k)
    assert torch.equal(r.topk_idx.cpu().long(), ref["topk_idx"])
    assert torch.equal(r.perm.cpu().long(), ref["perm"])
    assert torch.equal(r.inv_perm.cpu().long(), ref["inv_perm"])
    assert torch.equal(r.row_token.cpu().long(), ref["row_token"])
    assert torch.equal(r.offsets.cpu().long(), ref["offsets"])
    assert torch.allclose(r.topk_w.cpu(), ref["topk_w"], rtol=1e-5, atol=1e-7)
    counts = ref["offsets"][1:] - ref["offsets"][:-1]
    assert r.tile_prefix.cpu().tolist() == [0] + torch.div(counts + 255, 256, rounding_mode="floor").cumsum(0).tolist()
    assert r.blk_prefix.cpu().tolist() == [0] + torch.div(counts + 15, 16, rounding_mode="floor").cumsum(0).tolist()
    return r, ref


@pytest.mark.parametrize("T,E,k", [(64, 8, 2), (1000, 128, 8), (8192, 128, 8), (300, 5, 5), (2048, 200, 3)])
def test_route_bit_exact(artk_lib, gpu, T, E, k):
    print(f"moe route T={T} E={E} k={k}", flush=True)
    g = torch.Generator().manual_seed(T + E)
    check_routing(torch.randn(T, E, generator=g), k, gpu)


def test_route_ties_and_empty_experts(artk_lib, gpu):
    logits = torch.zeros(37, 16)          # all ties: every token picks experts 0..3
    logits[:, 9] = 1.0                    # ... except expert 9 first
    r, ref = check_routing(logits, 4, gpu)
    assert ref["topk_idx"][0].tolist() == [9, 0, 1, 2]
    assert (r.offsets.cpu()[4:9] == r.offsets.cpu()[4]).all()  # experts 3..8 empty


def test_route_nan_and_masked_logits(artk_lib, gpu):
    """Rows that are all NaN, or have fewer than k logits above -inf (masked experts, a diverged
    router), still give expert indices in [0, E): NaN counts as -inf, ties go to the lower index."""
    print("moe route with NaN / -inf rows", flush=True)
    g = torch.Generator().manual_seed(5)
    T, E, k = 517, 128, 8
    logits = torch.randn(T, E, generator=g)
    logits[3] = float("nan")
    logits[7] = float("-inf")
    logits[11, 5:] = float("-inf")               # 5 finite logits, k = 8
    logits[12, ::3] = float("nan")
    logits[13, :] = float("-inf")
    logits[13, 100] = 0.25                       # one finite logit
    logits[200:260, 64:] = float("-inf")         # half of the experts masked
    r, ref = check_routing(logits, k, gpu)
    idx = r.topk_idx.cpu()
    assert int(idx.min()) >= 0 and int(idx.max()) < E
    assert idx[3].tolist() == list(range(8)) and r.topk_w.cpu()[3].abs().max().item() == 0.0
    assert idx[13, 0].item() == 100 and r.topk_w.cpu()[13].tolist() == [1.0] + [0.0] * 7
    assert not torch.isnan(r.topk_w.cpu()).any()
    # one lane group past E (E = 200 leaves lanes of the fourth group without an expert)
    logits = torch.randn(64, 200, generator=g)
    logits[5] = float("nan")
    logits[6, 3:] = float("-inf")
    check_routing(logits, 5, gpu)


def make_experts(E, n_out, n_in, r, seed):
    g = torch.Generator().manual_seed(seed)
    W = (0.02 * torch.randn(E, n_out, n_in, generator=g)).to(torch.bfloat16)
    A = ((torch.rand(E, r, n_in, generator=g) * 2 - 1) / n_in ** 0.5).to(torch.bfloat16)
    B = (0.01 * torch.randn(E, n_out, r, generator=g)).to(torch.bfloat16)
    return W, A, B


@pytest.mark.parametrize("T,H,I,E,k,use_gather", [(256, 128, 64, 8, 2, True), (300, 192, 320, 16, 4, True),
                                                  (512, 128, 256, 8, 2, False), (64, 64, 64, 32, 8, True)])
def test_grouped_lora_matches_oracle(artk_lib, gpu, T, H, I, E, k, use_gather):
    print(f"moe grouped T={T} H={H} I={I} E={E} k={k} gather={use_gather}", flush=True)
    g = torch.Generator().manual_seed(T + I)
    logits = torch.randn(T, E, generator=g)
    r, ref = check_routing(logits, k, gpu)
    n_rows = T * k
    x = torch.randn(T if use_gather else n_rows, H, generator=g).to(torch.bfloat16)
    W, A, B = make_experts(E, I, H, 8, 3)
    up = torch.randn(n_rows, I, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(
        x, ref["row_token"] if use_gather else None, W, A, B, 2.0, ref["offsets"], up)
    gather = r.row_token if use_gather else None
    y, xa = ops.moe_lora_grouped_fwd(x.to(gpu), gather, W.to(gpu), A.to(gpu), B.to(gpu), 2.0, r)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), x.to(gpu), gather, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 2.0, r)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    if use_gather:  # oracle dx is per token; sum the kernel's per-row dx over each token's k rows
        dx = dx[r.inv_perm.long()].view(T, k, H).float().sum(1)
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL


@pytest.mark.parametrize("r,use_gather", [(40, True), (64, False), (16, True)])
def test_grouped_lora_ranks(artk_lib, gpu, r, use_gather):
    """Ranks other than 8: above 32 the one-pass backward runs its two-tile-per-rank shape (256-column
    chunks, two stages), with and without the row gather."""
    print(f"moe grouped rank {r} gather={use_gather}", flush=True)
    T, H, I, E, k = 384, 320, 192, 8, 2
    g = torch.Generator().manual_seed(100 + r)
    logits = torch.randn(T, E, generator=g)
    rt, ref = check_routing(logits, k, gpu)
    n_rows = T * k
    x = torch.randn(T if use_gather else n_rows, H, generator=g).to(torch.bfloat16)
    W, A, B = make_experts(E, I, H, r, 11)
    up = torch.randn(n_rows, I, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(
        x, ref["row_token"] if use_gather else None, W, A, B, 0.5, ref["offsets"], up)
    gather = rt.row_token if use_gather else None
    y, xa = ops.moe_lora_grouped_fwd(x.to(gpu), gather, W.to(gpu), A.to(gpu), B.to(gpu), 0.5, rt)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), x.to(gpu), gather, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 0.5, rt)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    if use_gather:
        dx = dx[rt.inv_perm.long()].view(T, k, H).float().sum(1)
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL


@pytest.mark.parametrize("use_gather", [True, False])
def test_grouped_lora_with_empty_experts(artk_lib, gpu, use_gather):
    """Experts that no token chose: their dA_e and dB_e are exactly zero, the others match the oracle
    (the one-pass backward gives every expert its own slab of rows, here some of them empty, one of
    them longer than a 128-row tile and the first and last expert among the empty ones)."""
    print(f"moe grouped, empty experts, gather={use_gather}", flush=True)
    T, H, I, E, k = 320, 128, 192, 16, 2
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g)
    dead = [0, 3, 4, 5, 15]
    logits[:, dead] = float("-inf")
    logits[:200, 7] += 8.0                      # expert 7 gets at least 200 rows
    r, ref = check_routing(logits, k, gpu)
    off = ref["offsets"]
    assert all(off[e + 1] == off[e] for e in dead) and off[8] - off[7] >= 200
    n_rows = T * k
    x = torch.randn(T if use_gather else n_rows, H, generator=g).to(torch.bfloat16)
    W, A, B = make_experts(E, I, H, 8, 9)
    up = torch.randn(n_rows, I, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(
        x, ref["row_token"] if use_gather else None, W, A, B, 2.0, off, up)
    gather = r.row_token if use_gather else None
    y, xa = ops.moe_lora_grouped_fwd(x.to(gpu), gather, W.to(gpu), A.to(gpu), B.to(gpu), 2.0, r)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), x.to(gpu), gather, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 2.0, r)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    if use_gather:
        dx = dx[r.inv_perm.long()].view(T, k, H).float().sum(1)
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL and rel_l2(dB.cpu(), dB0) <= TOL
    for e in dead:
        assert dA[e].abs().max().item() == 0.0 and dB[e].abs().max().item() == 0.0
    for e in (7, 8):
        assert rel_l2(dA[e].cpu(), dA0[e]) <= TOL and rel_l2(dB[e].cpu(), dB0[e]) <= TOL


def test_config5_gate_projection_full_size(artk_lib, gpu):
    """Benchmark config 5: 8192 tokens, hidden 2048, 128 experts, top-8, gate [768,2048]."""
    print("moe config5 gate projection", flush=True)
    T, H, I, E, k = 8192, 2048, 768, 128, 8
    g = torch.Generator().manual_seed(1005)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    r, ref = check_routing(logits, k, gpu)
    W, A, B = make_experts(E, I, H, 8, 1005)
    up = torch.randn(T * k, I, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(x, ref["row_token"], W, A, B, 2.0, ref["offsets"], up)
    y, xa = ops.moe_lora_grouped_fwd(x.to(gpu), r.row_token, W.to(gpu), A.to(gpu), B.to(gpu), 2.0, r)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), x.to(gpu), r.row_token, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 2.0, r)
    dx = dx[r.inv_perm.long()].view(T, k, H).float().sum(1)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL


def test_config5_down_projection_full_size(artk_lib, gpu):
    """Benchmark config 5, down projection [2048,768] at full size: 65536 sorted rows of width 768
    (no gather: the rows are the gated activations, already in expert order), forward and backward."""
    print("moe config5 down projection", flush=True)
    T, H, I, E, k = 8192, 2048, 768, 128, 8
    g = torch.Generator().manual_seed(1005)
    logits = torch.randn(T, E, generator=g)
    r, ref = check_routing(logits, k, gpu)
    h = torch.randn(T * k, I, generator=g).to(torch.bfloat16)
    W, A, B = make_experts(E, H, I, 8, 2005)
    up = torch.randn(T * k, H, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(h, None, W, A, B, 2.0, ref["offsets"], up)
    y, xa = ops.moe_lora_grouped_fwd(h.to(gpu), None, W.to(gpu), A.to(gpu), B.to(gpu), 2.0, r)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), h.to(gpu), None, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 2.0, r)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL
    # per expert as well: a wrong expert boundary would hide in the global norm
    off = ref["offsets"].tolist()
    for e in (0, 1, 63, 127):
        sl = slice(off[e], off[e + 1])
        assert rel_l2(y[sl].cpu().float(), y0[sl]) <= TOL
        assert rel_l2(dx[sl].cpu().float(), dx0[sl]) <= TOL
        assert rel_l2(dA[e].cpu(), dA0[e]) <= TOL and rel_l2(dB[e].cpu(), dB0[e]) <= TOL


def test_config5_fused_gate_up_full_size(artk_lib, gpu):
    """Benchmark config 5 the way art_amd.moe.MoELoRAExperts runs gate and up: ONE grouped product
    [128, 1536, 2048] over the gathered token rows, adapters stacked to rank 16 with a block-diagonal
    B per expert.  y, dx (summed per token), dA and dB against the oracle, also expert by expert;
    gate and up halves against the oracle of each projection alone."""
    print("moe config5 fused gate|up", flush=True)
    T, H, I, E, k, r = 8192, 2048, 768, 128, 8, 8
    g = torch.Generator().manual_seed(1005)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    rt, ref = check_routing(logits, k, gpu)
    Wg, Ag, Bg = make_experts(E, I, H, r, 1005)
    Wu, Au, Bu = make_experts(E, I, H, r, 3005)
    W = torch.cat([Wg, Wu], 1).contiguous()
    A = torch.cat([Ag, Au], 1).contiguous()
    B = torch.zeros(E, 2 * I, 2 * r, dtype=torch.bfloat16)
    B[:, :I, :r], B[:, I:, r:] = Bg, Bu
    up = torch.randn(T * k, 2 * I, generator=g).to(torch.bfloat16)
    y0, dx0, dA0, dB0 = moe_oracle.grouped_lora_grads(x, ref["row_token"], W, A, B, 2.0, ref["offsets"], up)
    y, xa = ops.moe_lora_grouped_fwd(x.to(gpu), rt.row_token, W.to(gpu), A.to(gpu), B.to(gpu), 2.0, rt)
    dx, dA, dB = ops.moe_lora_grouped_bwd(up.to(gpu), x.to(gpu), rt.row_token, ops.transpose_batched(W.to(gpu)),
                                          A.to(gpu), B.to(gpu), xa, 2.0, rt)
    dx = dx[rt.inv_perm.long()].view(T, k, H).float().sum(1)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL
    off = ref["offsets"].tolist()
    for e in (0, 1, 63, 127):
        sl = slice(off[e], off[e + 1])
        assert rel_l2(y[sl].cpu().float(), y0[sl]) <= TOL
        assert rel_l2(dA[e].cpu(), dA0[e]) <= TOL and rel_l2(dB[e].cpu(), dB0[e]) <= TOL
    # the halves are the two projections: forward and adapter gradients of gate alone
    yg0, _, dAg0, dBg0 = moe_oracle.grouped_lora_grads(x, ref["row_token"], Wg, Ag, Bg, 2.0, ref["offsets"],
                                                        up[:, :I].contiguous())
    assert rel_l2(y[:, :I].cpu().float(), yg0) <= TOL
    assert rel_l2(dA[:, :r].cpu(), dAg0) <= TOL
    assert rel_l2(dB[:, :I, :r].cpu(), dBg0) <= TOL


def test_moe_block_autograd(artk_lib, gpu):
    """The whole block (gate, up, SiLU gating, down, recombination) against torch fp32."""
    torch.manual_seed(0)
    T, H, I, E, k = 192, 128, 64, 8, 2
    mod = MoELoRAExperts(H, I, E, k, device=gpu)
    with torch.no_grad():
        for n in ("gate", "up", "down"):
            getattr(mod, f"{n}_lora_B").normal_(std=0.02)
    x = torch.randn(T, H, device=gpu).to(torch.bfloat16).requires_grad_(True)
    logits = torch.randn(T, E, device=gpu)
    y, routing = mod(x, logits)
    up = torch.randn_like(y)
    y.backward(up)
    # reference: dense per-token evaluation in fp32 on the CPU
    ref = moe_oracle.route(logits.cpu(), k)
    xr = x.detach().cpu().float().requires_grad_(True)
    P = {n: p.detach().cpu().float().requires_grad_(p.requires_grad) for n, p in mod.named_parameters()}
    assert "gate_weight" not in P and "up_weight" not in P    # one stored weight; gate / up are views of it
    assert mod.gate_weight.data_ptr() == mod.gate_up_weight.data_ptr()
    P["gate_weight"], P["up_weight"] = P["gate_up_weight"][:, :I], P["gate_up_weight"][:, I:]
    rows = xr[ref["row_token"]]
    off = ref["offsets"]
    s = mod.scaling
    gate = moe_oracle.grouped_lora(rows, P["gate_weight"], P["gate_lora_A"], P["gate_lora_B"], s, off)
    upp = moe_oracle.grouped_lora(rows, P["up_weight"], P["up_lora_A"], P["up_lora_B"], s, off)
    h = torch.nn.functional.silu(gate) * upp
    down = moe_oracle.grouped_lora(h, P["down_weight"], P["down_lora_A"], P["down_lora_B"], s, off)
    y0 = (down[ref["inv_perm"]].view(T, k, H) * ref["topk_w"].unsqueeze(-1)).sum(1)
    y0.backward(up.cpu().float())
    assert rel_l2(y.detach().cpu().float(), y0.detach()) <= 2e-2
    assert rel_l2(x.grad.cpu().float(), xr.grad) <= 2e-2
    for n in ("gate_lora_A", "gate_lora_B", "up_lora_A", "up_lora_B", "down_lora_A", "down_lora_B"):
        assert rel_l2(getattr(mod, n).grad.cpu(), P[n].grad) <= 2e-2, n
