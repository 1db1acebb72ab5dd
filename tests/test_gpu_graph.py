"""The library calls launch on the caller's stream, never synchronise and
allocate nothing themselves, so a caller can record them into a HIP graph.
Each replay runs with new contents in the static input buffers, with eager work
and synchronisations in between, and is compared bit for bit with the eager
result on the same inputs."""
import os
import sys

import pytest
import torch

from art_amd import ops, synthetic

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager(artk_lib, gpu):
    T, H, V = 512, 128, 4096
    cases = [synthetic.make_grpo_case("g", 50 + i, T, H, V, 4, 4, 0.5) for i in range(3)]
    for c in cases:
        new, _ = ops.logprob_fwd(c.hidden.view(T, H).to(gpu), c.lm_head.to(gpu), c.tokens.view(T).to(gpu), True, T)
        c.finish(new.cpu())
    lm_head = cases[0].lm_head.to(gpu)
    lm_head_t = ops.transpose(lm_head)
    S, Hq, Hkv, D = 256, 2, 1, 64
    group, parent = synthetic.packed_row_ids(3, S, 1, 32, 4, 56)
    plan = ops.attn_plan(group.to(gpu), parent.to(gpu))
    n_in, n_out, r = 128, 256, 8
    g = torch.Generator().manual_seed(1)
    W = (0.02 * torch.randn(n_out, n_in, generator=g)).to(torch.bfloat16).to(gpu)
    A = (0.05 * torch.randn(r, n_in, generator=g)).to(torch.bfloat16).to(gpu)
    B = (0.05 * torch.randn(n_out, r, generator=g)).to(torch.bfloat16).to(gpu)

    # static inputs of the graph
    st = {
        "hidden": torch.empty(T, H, dtype=torch.bfloat16, device=gpu),
        "tokens": torch.empty(T, dtype=torch.int64, device=gpu),
        "old": torch.empty(T, dtype=torch.float32, device=gpu),
        "adv": torch.empty(T, dtype=torch.float32, device=gpu),
        "mask": torch.empty(T, dtype=torch.bool, device=gpu),
        "w": torch.empty(T, dtype=torch.float32, device=gpu),
        "q": torch.empty(S, Hq, D, dtype=torch.bfloat16, device=gpu),
        "k": torch.empty(S, Hkv, D, dtype=torch.bfloat16, device=gpu),
        "v": torch.empty(S, Hkv, D, dtype=torch.bfloat16, device=gpu),
    }

    def load(i):
        c = cases[i]
        st["hidden"].copy_(c.hidden.view(T, H))
        st["tokens"].copy_(c.tokens.view(T))
        st["old"].copy_(c.logprobs.view(T))
        st["adv"].copy_(c.advantages.view(T))
        st["mask"].copy_(c.assistant_mask.view(T))
        st["w"].copy_(c.weights.view(T))
        gq = torch.Generator().manual_seed(100 + i)
        for name in ("q", "k", "v"):
            st[name].copy_(torch.randn(st[name].shape, generator=gq).to(torch.bfloat16))

    def run():
        s, lp, dh = ops.grpo_fused(st["hidden"], lm_head, lm_head_t, st["tokens"], st["old"], st["adv"],
                                   st["mask"], st["w"], None, T, 0.8, 1.2, 0.0, 256)
        y, xa = ops.lora_linear_fwd(st["hidden"], W, A, B, 2.0)
        out, lse = ops.attn_fwd(st["q"], st["k"], st["v"], plan)
        return s, lp, dh, y, out, lse

    load(0)
    eager = [[t.clone() for t in run()]]
    for i in (1, 2):
        load(i)
        eager.append([t.clone() for t in run()])
    torch.cuda.synchronize()

    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run()
    for i in (0, 1, 2, 1):
        load(i)
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager[i]):
            assert torch.equal(got.nan_to_num(0.0), want.nan_to_num(0.0))
        _ = (st["hidden"].float() @ st["hidden"].float().t()).sum().item()  # eager work between replays
