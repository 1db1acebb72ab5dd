"""GPU parity of the LoRA linear (forward and backward) against the CPU oracle.

Tolerance: rel-L2 <= 1e-2 for y, dx, dA, dB against the fp32 oracle evaluated
on the same bf16-valued inputs."""
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import lora_oracle  # noqa: E402

from art_amd import ops  # noqa: E402
from art_amd.lora import LoRALinear, lora_linear  # noqa: E402

pytestmark = pytest.mark.gpu
TOL = 1e-2


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def make(T, n_in, n_out, r, seed, b_std=0.01):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, n_in, generator=g).to(torch.bfloat16)
    W = (0.02 * torch.randn(n_out, n_in, generator=g)).to(torch.bfloat16)
    bound = 1.0 / math.sqrt(n_in)  # Kaiming-uniform with a = sqrt(5)
    A = ((torch.rand(r, n_in, generator=g) * 2 - 1) * bound).to(torch.bfloat16)
    B = (b_std * torch.randn(n_out, r, generator=g)).to(torch.bfloat16)
    up = torch.randn(T, n_out, generator=g).to(torch.bfloat16)
    return x, W, A, B, up


def run_gpu(x, W, A, B, up, scale, gpu):
    xd, Wd, Ad, Bd, upd = (t.to(gpu) for t in (x, W, A, B, up))
    y, xa = ops.lora_linear_fwd(xd, Wd, Ad, Bd, scale)
    dx, dA, dB = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    return y.cpu().float(), dx.cpu().float(), dA.cpu(), dB.cpu()


@pytest.mark.parametrize("T,n_in,n_out,r", [(512, 256, 256, 8), (300, 192, 320, 8), (256, 128, 64, 16),
                                            (1000, 512, 576, 24),
                                            (5000, 192, 4160, 8)])  # more tiles than CUs, ragged on both sides
def test_lora_matches_oracle(artk_lib, gpu, T, n_in, n_out, r):
    print(f"lora T={T} in={n_in} out={n_out} r={r}", flush=True)
    x, W, A, B, up = make(T, n_in, n_out, r, T + r)
    scale = 16 / r
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, scale, up)
    y, dx, dA, dB = run_gpu(x, W, A, B, up, scale, gpu)
    assert rel_l2(y, y0) <= TOL
    assert rel_l2(dx, dx0) <= TOL
    assert rel_l2(dA, dA0) <= TOL
    assert rel_l2(dB, dB0) <= TOL


def test_lora_zero_factors(artk_lib, gpu):
    """B = 0: y is the base projection and dA vanishes; A = 0: dB vanishes."""
    x, W, A, B, up = make(256, 128, 192, 8, 5)
    y, dx, dA, dB = run_gpu(x, W, A, torch.zeros_like(B), up, 2.0, gpu)
    base = ops.gemm_nt(W.to(gpu), x.to(gpu)).cpu().float()
    assert torch.equal(y, base)
    assert dA.abs().max().item() == 0.0
    assert dB.abs().max().item() > 0.0
    y, dx, dA, dB = run_gpu(x, W, torch.zeros_like(A), B, up, 2.0, gpu)
    assert dB.abs().max().item() == 0.0
    assert dA.abs().max().item() > 0.0


@pytest.mark.parametrize("n_out", [2048, 256, 11008])
def test_lora_config2_full_size(artk_lib, gpu, n_out):
    """Benchmark config 2 (Qwen2.5-3B projections) at full size."""
    print(f"lora config2 out={n_out}", flush=True)
    x, W, A, B, up = make(8192, 2048, n_out, 8, 1002 + n_out)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, 2.0, up)
    y, dx, dA, dB = run_gpu(x, W, A, B, up, 2.0, gpu)
    assert rel_l2(y, y0) <= TOL
    assert rel_l2(dx, dx0) <= TOL
    assert rel_l2(dA, dA0) <= TOL
    assert rel_l2(dB, dB0) <= TOL


def test_lora_down_projection_full_size(artk_lib, gpu):
    """The seventh target module of the reference's adapter config (down_proj, 11008 -> 2048,
    src/art/dev/model.py:54-62) at full size, with rank 16."""
    print("lora down_proj 11008 -> 2048, r=16", flush=True)
    x, W, A, B, up = make(4096, 11008, 2048, 16, 1717)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, 1.0, up)
    y, dx, dA, dB = run_gpu(x, W, A, B, up, 1.0, gpu)
    assert rel_l2(y, y0) <= TOL
    assert rel_l2(dx, dx0) <= TOL
    assert rel_l2(dA, dA0) <= TOL
    assert rel_l2(dB, dB0) <= TOL


def test_lora_module_autograd(artk_lib, gpu):
    torch.manual_seed(0)
    mod = LoRALinear(256, 320, r=8, lora_alpha=16, device=gpu, dtype=torch.float32)
    with torch.no_grad():
        mod.lora_B.normal_(std=0.01)
    x = torch.randn(2, 96, 256, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    y = mod(x)
    assert y.shape == (2, 96, 320)
    up = torch.randn_like(y)
    y.backward(up)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(
        x.detach().cpu().view(-1, 256), mod.weight.cpu(), mod.lora_A.detach().cpu().to(torch.bfloat16),
        mod.lora_B.detach().cpu().to(torch.bfloat16), mod.scaling, up.cpu().view(-1, 320))
    assert rel_l2(y.detach().cpu().float().view(-1, 320), y0) <= TOL
    assert rel_l2(x.grad.cpu().float().view(-1, 256), dx0) <= TOL
    assert rel_l2(mod.lora_A.grad.cpu(), dA0) <= TOL
    assert rel_l2(mod.lora_B.grad.cpu(), dB0) <= TOL
    assert mod.weight.grad is None


def test_fused_projections_match_separate(artk_lib, gpu):
    """q/k/v as one product: same outputs and gradients as three LoRALinear modules."""
    from art_amd.lora import FusedLoRALinear, LoRALinear
    torch.manual_seed(5)
    T, n_in = 192, 256
    layers = [LoRALinear(n_in, o, r=8, lora_alpha=16, device=gpu, dtype=torch.float32) for o in (256, 64, 64)]
    for l in layers:
        torch.nn.init.normal_(l.lora_B, std=0.05)
    fused = FusedLoRALinear(layers)
    x1 = torch.randn(T, n_in, device=gpu).to(torch.bfloat16).requires_grad_(True)
    x2 = x1.detach().clone().requires_grad_(True)
    ups = [torch.randn(T, o, device=gpu).to(torch.bfloat16) for o in (256, 64, 64)]
    ys = [l(x1) for l in layers]
    sum((y.float() * u.float()).sum() for y, u in zip(ys, ups)).backward()
    ref = [(l.lora_A.grad.clone(), l.lora_B.grad.clone()) for l in layers]
    for l in layers:
        l.lora_A.grad = None
        l.lora_B.grad = None
    yf = fused(x2)
    sum((y.float() * u.float()).sum() for y, u in zip(yf, ups)).backward()
    rel = lambda a, b: ((a.double() - b.double()).norm() / b.double().norm()).item()
    for a, b in zip(yf, ys):
        assert rel(a.float(), b.float()) <= 4e-3
    assert rel(x2.grad.float(), x1.grad.float()) <= 1e-2
    for l, (dA, dB) in zip(layers, ref):
        assert rel(l.lora_A.grad, dA) <= 1e-2 and rel(l.lora_B.grad, dB) <= 1e-2


@pytest.mark.parametrize("n_out,r", [(2048, 8), (256, 8), (320, 48)])
def test_lora_bias_and_ranks(artk_lib, gpu, n_out, r):
    """Qwen2.5's q/k/v projections carry a (frozen) bias: y = x W^T + bias + s (x A^T) B^T at the
    config-2 q and k/v shapes, and a rank above 32 on a ragged shape (two e tiles in the
    one-pass skinny products).  The bias adds nothing to dx, dA, dB."""
    print(f"lora bias out={n_out} r={r}", flush=True)
    T, n_in = (8192, 2048) if r == 8 else (1100, 448)
    x, W, A, B, up = make(T, n_in, n_out, r, 77 + n_out)
    bias = (0.5 * torch.randn(n_out, generator=torch.Generator().manual_seed(n_out))).to(torch.bfloat16)
    scale = 16 / r
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, scale, up)
    y0 = y0 + bias.float()
    xd, Wd, Ad, Bd, upd = (t.to(gpu) for t in (x, W, A, B, up))
    y, xa = ops.lora_linear_fwd(xd, Wd, Ad, Bd, scale, bias.to(gpu))
    dx, dA, dB = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    assert rel_l2(y.cpu().float(), y0) <= TOL
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    assert rel_l2(dA.cpu(), dA0) <= TOL
    assert rel_l2(dB.cpu(), dB0) <= TOL
    # bit-reproducible run to run (fixed summation orders)
    dx2, dA2, dB2 = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    assert torch.equal(dA, dA2) and torch.equal(dB, dB2) and torch.equal(dx, dx2)


def test_lora_module_with_bias_from_linear(artk_lib, gpu):
    """LoRALinear.from_linear keeps the base layer's bias (as peft does) and leaves it frozen."""
    torch.manual_seed(3)
    lin = torch.nn.Linear(256, 192, bias=True, device=gpu, dtype=torch.bfloat16)
    mod = LoRALinear.from_linear(lin, r=8, lora_alpha=16)
    assert mod.bias is not None and not mod.bias.requires_grad
    with torch.no_grad():
        mod.lora_B.normal_(std=0.02)
    x = torch.randn(300, 256, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    y = mod(x)
    y.backward(torch.ones_like(y))
    want = (x.detach().float() @ lin.weight.float().t() + lin.bias.float()
            + mod.scaling * (x.detach().float() @ mod.lora_A.float().t()) @ mod.lora_B.float().t())
    assert rel_l2(y.detach().float().cpu(), want.cpu()) <= TOL
    assert mod.bias.grad is None and mod.lora_A.grad is not None


# ---- projections of the same input in one call (q|k|v, gate|up) ------------------------------------
_oracle_cache = {}


def shared_input_case(T, n_in, outs, ranks, seed, with_bias):
    """Per projection (W, A, B, bias, g) on one x, and the oracle's (y, dx, dA, dB) of each."""
    key = (T, n_in, tuple(outs), tuple(ranks), seed, with_bias)
    if key not in _oracle_cache:
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(T, n_in, generator=g).to(torch.bfloat16)
        parts, refs = [], []
        for o, r in zip(outs, ranks):
            W = (0.02 * torch.randn(o, n_in, generator=g)).to(torch.bfloat16)
            A = ((torch.rand(r, n_in, generator=g) * 2 - 1) / math.sqrt(n_in)).to(torch.bfloat16)
            B = (0.01 * torch.randn(o, r, generator=g)).to(torch.bfloat16)
            bias = (0.5 * torch.randn(o, generator=g)).to(torch.bfloat16) if with_bias else None
            up = torch.randn(T, o, generator=g).to(torch.bfloat16)
            parts.append((W, A, B, bias, up))
        scale = 16 / ranks[0]
        for W, A, B, bias, up in parts:
            y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x, W, A, B, scale, up)
            refs.append((y0 + bias.float() if with_bias else y0, dx0, dA0, dB0))
        _oracle_cache.clear()          # one case at a time: a gate|up case holds 3 GB of fp32 references
        _oracle_cache[key] = (x, parts, refs, scale)
    return _oracle_cache[key]


MULTI_CASES = [
    pytest.param(8192, 2048, (2048, 256, 256), (8, 8, 8), True, id="c2-qkv"),
    pytest.param(8192, 2048, (11008, 11008), (8, 8), False, id="c2-gate_up"),
    pytest.param(300, 192, (320, 64), (16, 16), True, id="ragged"),
    pytest.param(1000, 448, (192, 576, 64, 128), (8, 8, 8, 8), False, id="four"),
]


@pytest.mark.parametrize("T,n_in,outs,ranks,with_bias", MULTI_CASES)
def test_multi_projection_matches_oracle(artk_lib, gpu, T, n_in, outs, ranks, with_bias):
    """artk_lora_linear_multi_fwd / _bwd (separate weights, adapters, outputs and upstream gradients)
    against the oracle evaluated projection by projection; dx is the sum over the projections.  The
    two config-2 cases are the call shapes of a Qwen2.5-3B layer at full size."""
    print(f"lora multi T={T} in={n_in} outs={outs} ranks={ranks}", flush=True)
    x, parts, refs, scale = shared_input_case(T, n_in, outs, ranks, 4242 + T, with_bias)
    xd = x.to(gpu)
    Ws = [p[0].to(gpu) for p in parts]
    As = [p[1].to(gpu) for p in parts]
    Bs = [p[2].to(gpu) for p in parts]
    biases = [p[3].to(gpu) for p in parts] if with_bias else None
    gs = [p[4].to(gpu) for p in parts]
    ys, xas = ops.lora_linear_multi_fwd(xd, Ws, As, Bs, scale, biases)
    dx, dAs, dBs = ops.lora_linear_multi_bwd(gs, xd, [ops.transpose(w) for w in Ws], As, Bs, xas, scale)
    dx0 = sum(r[1] for r in refs)
    assert rel_l2(dx.cpu().float(), dx0) <= TOL
    for i, (y0, _, dA0, dB0) in enumerate(refs):
        assert rel_l2(ys[i].cpu().float(), y0) <= TOL, i
        assert rel_l2(dAs[i].cpu(), dA0) <= TOL, i
        assert rel_l2(dBs[i].cpu(), dB0) <= TOL, i
    # bit-reproducible run to run, and identical to the single-projection entry points on each projection's
    # own outputs (same kernels and summation orders; dx differs: it is one accumulation here)
    dx2, dAs2, dBs2 = ops.lora_linear_multi_bwd(gs, xd, [ops.transpose(w) for w in Ws], As, Bs, xas, scale)
    assert torch.equal(dx, dx2) and all(torch.equal(a, b) for a, b in zip(dAs + dBs, dAs2 + dBs2))
    y_one, xa_one = ops.lora_linear_fwd(xd, Ws[-1], As[-1], Bs[-1], scale, None if biases is None else biases[-1])
    assert torch.equal(y_one, ys[-1]) and torch.equal(xa_one, xas[-1])


@pytest.mark.parametrize("T,n_in,outs,ranks,with_bias", MULTI_CASES[:2])
def test_concatenated_projections_config2_full_size(artk_lib, gpu, T, n_in, outs, ranks, with_bias):
    """The single-projection entry points on the concatenated form of the same cases: weights stacked
    along the output dimension, A stacked, B block-diagonal (out 2560 / rank 24 with the q, k, v biases;
    out 22016 / rank 16).  The diagonal blocks of dB are the adapters' gradients; the off-diagonal
    blocks are derivatives with respect to entries that are pinned to zero and belong to no adapter
    (they are not zero; they are checked against the oracle's full product like the rest)."""
    print(f"lora concatenated out={sum(outs)} r={sum(ranks)}", flush=True)
    x, parts, refs, scale = shared_input_case(T, n_in, outs, ranks, 4242 + T, with_bias)
    W = torch.cat([p[0] for p in parts], 0)
    A = torch.cat([p[1] for p in parts], 0)
    B = torch.zeros(sum(outs), sum(ranks), dtype=torch.bfloat16)
    o0 = r0 = 0
    for (p, o, r) in zip(parts, outs, ranks):
        B[o0:o0 + o, r0:r0 + r] = p[2]
        o0, r0 = o0 + o, r0 + r
    bias = torch.cat([p[3] for p in parts]) if with_bias else None
    up = torch.cat([p[4] for p in parts], 1)
    xd, Wd, Ad, Bd, upd = (t.to(gpu).contiguous() for t in (x, W, A, B, up))
    y, xa = ops.lora_linear_fwd(xd, Wd, Ad, Bd, scale, None if bias is None else bias.to(gpu))
    dx, dA, dB = ops.lora_linear_bwd(upd, xd, ops.transpose(Wd), Ad, Bd, xa, scale)
    assert rel_l2(dx.cpu().float(), sum(r[1] for r in refs)) <= TOL
    o0 = r0 = 0
    for (y0, _, dA0, dB0), o, r in zip(refs, outs, ranks):
        assert rel_l2(y[:, o0:o0 + o].cpu().float(), y0) <= TOL
        assert rel_l2(dA[r0:r0 + r].cpu(), dA0) <= TOL
        assert rel_l2(dB[o0:o0 + o, r0:r0 + r].cpu(), dB0) <= TOL
        o0, r0 = o0 + o, r0 + r
    # the whole dB, off-diagonal blocks included: s g^T (x A_cat^T) in fp64 on the CPU
    xa0 = x.double() @ A.double().t()
    dB_full = scale * (up.double().t() @ xa0)
    assert rel_l2(dB.cpu(), dB_full) <= TOL
