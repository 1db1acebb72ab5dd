"""GPU parity of the NF4 dequantisation against the CPU oracle: bit-exact (table
look-up, one fp32 multiplication, round-to-nearest-even to bf16), in both the
plain and the double-quantised form; the quantiser of NF4Weight against the
oracle's; LoRA linear on a dequantised base weight."""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import quant_oracle as qo  # noqa: E402

from art_amd import ops  # noqa: E402
from art_amd.quant import NF4Weight  # noqa: E402

pytestmark = pytest.mark.gpu


def bits(t):
    return t.cpu().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("n,blocksize", [(64, 64), (64 * 777, 64), (128 * 100, 128), (32 * 5, 32)])
def test_dequant_bit_exact(artk_lib, gpu, n, blocksize):
    g = np.random.default_rng(n)
    packed = g.integers(0, 256, n // 2, dtype=np.uint8)
    absmax = np.abs(g.standard_normal(n // blocksize)).astype(np.float32) * 0.05
    want = qo.to_bf16_bits(qo.dequantize(packed, absmax, blocksize))
    got = ops.nf4_dequant(torch.from_numpy(packed).to(gpu), torch.from_numpy(absmax).to(gpu), blocksize=blocksize)
    assert np.array_equal(bits(got), want)


def test_dequant_double_quantised_bit_exact(artk_lib, gpu):
    g = np.random.default_rng(5)
    n, blocksize = 64 * 600, 64
    packed = g.integers(0, 256, n // 2, dtype=np.uint8)
    absmax_q = g.integers(0, 256, n // blocksize, dtype=np.uint8)
    code2 = np.sort(g.uniform(-1, 1, 256)).astype(np.float32)
    absmax2 = np.abs(g.standard_normal(3)).astype(np.float32)
    offset = 0.0371
    absmax = qo.nested_absmax(absmax_q, code2, absmax2, offset)
    want = qo.to_bf16_bits(qo.dequantize(packed, absmax, blocksize))
    t = lambda a: torch.from_numpy(a).to(gpu)
    got = ops.nf4_dequant(t(packed), None, t(absmax_q), t(code2), t(absmax2), offset, blocksize)
    assert np.array_equal(bits(got), want)


def test_quantiser_and_lora_on_nf4_base(artk_lib, gpu):
    g = torch.Generator().manual_seed(9)
    n_out, n_in, T, r = 256, 128, 64, 8
    W = 0.02 * torch.randn(n_out, n_in, generator=g)
    q = NF4Weight.from_float(W.to(gpu))
    packed, absmax = qo.quantize(W.numpy().reshape(-1), 64)
    assert np.array_equal(q.packed.cpu().numpy(), packed)
    assert np.array_equal(q.absmax.cpu().numpy(), absmax)
    Wd = q.dequantize()
    assert Wd.shape == (n_out, n_in) and torch.equal(q.dequantize_transposed(), Wd.t().contiguous())
    # y = x Wd^T + s (x A^T) B^T with the dequantised base weight
    x = torch.randn(T, n_in, generator=g).to(torch.bfloat16)
    A = (0.05 * torch.randn(r, n_in, generator=g)).to(torch.bfloat16)
    B = (0.05 * torch.randn(n_out, r, generator=g)).to(torch.bfloat16)
    y, _ = ops.lora_linear_fwd(x.to(gpu), Wd, A.to(gpu), B.to(gpu), 2.0)
    ref = x.float() @ Wd.float().cpu().t() + 2.0 * (x.float() @ A.float().t()) @ B.float().t()
    assert ((y.float().cpu() - ref).norm() / ref.norm()).item() <= 1e-2


@pytest.mark.parametrize("rows,cols,blocksize,nested", [(256, 128, 64, False), (11008, 2048, 64, False),
                                                        (200, 192, 32, True), (72, 64, 64, False)])
def test_dequant_transposed_bit_exact(artk_lib, gpu, rows, cols, blocksize, nested):
    """The transposed dequantisation writes exactly the values of the plain one, at [c, r]."""
    g = np.random.default_rng(rows + cols)
    n = rows * cols
    packed = torch.from_numpy(g.integers(0, 256, n // 2, dtype=np.uint8)).to(gpu)
    kw = {}
    if nested:
        kw = dict(absmax_q=torch.from_numpy(g.integers(0, 256, n // blocksize, dtype=np.uint8)).to(gpu),
                  code2=torch.from_numpy(np.sort(g.uniform(-1, 1, 256)).astype(np.float32)).to(gpu),
                  absmax2=torch.from_numpy(np.abs(g.standard_normal((n // blocksize + 255) // 256)).astype(np.float32)).to(gpu),
                  offset=0.0123)
    else:
        kw = dict(absmax=torch.from_numpy(np.abs(g.standard_normal(n // blocksize)).astype(np.float32) * 0.05).to(gpu))
    plain = ops.nf4_dequant(packed, blocksize=blocksize, **kw).view(rows, cols)
    tr = ops.nf4_dequant_t(packed, rows, cols, blocksize=blocksize, **kw)
    assert tr.shape == (cols, rows)
    assert torch.equal(tr, plain.t().contiguous())


@pytest.mark.parametrize("n_out,n_in,T,r,with_bias", [(256, 128, 64, 8, False), (2048, 2048, 1024, 8, True),
                                                      (320, 192, 300, 16, True)])
def test_lora_on_nf4_weight_without_resident_copies(artk_lib, gpu, n_out, n_in, T, r, with_bias):
    """artk_lora_linear_fwd_nf4 / _bwd_nf4 (the 16-bit weight exists only inside the call) give,
    bit for bit, what the bf16 entry points give on the dequantised weight and its transposed
    copy; and the result is the LoRA linear of the oracle on that weight."""
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
    import lora_oracle

    print(f"lora on NF4 weight out={n_out} in={n_in} T={T} r={r}", flush=True)
    g = torch.Generator().manual_seed(n_out + T)
    q = NF4Weight.from_float((0.02 * torch.randn(n_out, n_in, generator=g)).to(gpu))
    x = torch.randn(T, n_in, generator=g).to(torch.bfloat16).to(gpu)
    A = (0.05 * torch.randn(r, n_in, generator=g)).to(torch.bfloat16).to(gpu)
    B = (0.05 * torch.randn(n_out, r, generator=g)).to(torch.bfloat16).to(gpu)
    up = torch.randn(T, n_out, generator=g).to(torch.bfloat16).to(gpu)
    bias = (0.3 * torch.randn(n_out, generator=g)).to(torch.bfloat16).to(gpu) if with_bias else None
    y, xa = ops.lora_linear_fwd_nf4(x, q, A, B, 2.0, bias)
    dx, dA, dB = ops.lora_linear_bwd_nf4(up, x, q, A, B, xa, 2.0)
    Wd = q.dequantize()
    y2, xa2 = ops.lora_linear_fwd(x, Wd, A, B, 2.0, bias)
    dx2, dA2, dB2 = ops.lora_linear_bwd(up, x, ops.transpose(Wd), A, B, xa2, 2.0)
    for a, b in ((y, y2), (xa, xa2), (dx, dx2), (dA, dA2), (dB, dB2)):
        assert torch.equal(a, b)
    y0, dx0, dA0, dB0 = lora_oracle.lora_linear_grads(x.cpu(), Wd.cpu(), A.cpu(), B.cpu(), 2.0, up.cpu())
    if bias is not None:
        y0 = y0 + bias.float().cpu()
    rel = lambda a, b: ((a.double().cpu() - b.double()).norm() / b.double().norm()).item()
    assert rel(y, y0) <= 1e-2 and rel(dx, dx0) <= 1e-2 and rel(dA, dA0) <= 1e-2 and rel(dB, dB0) <= 1e-2


def test_lora_module_from_nf4(artk_lib, gpu):
    """LoRALinear.from_nf4 holds the 4-bit form only and trains its adapters through it."""
    from art_amd.lora import LoRALinear

    torch.manual_seed(4)
    W = 0.02 * torch.randn(192, 256)
    q = NF4Weight.from_float(W.to(gpu))
    mod = LoRALinear.from_nf4(q, r=8, lora_alpha=16)
    assert mod.weight is None and sum(p.numel() for p in mod.parameters()) == 8 * (192 + 256)
    with torch.no_grad():
        mod.lora_B.normal_(std=0.02)
    x = torch.randn(130, 256, device=gpu, dtype=torch.bfloat16, requires_grad=True)
    y = mod(x)
    y.backward(torch.ones_like(y))
    Wd = q.dequantize().float()
    want = x.detach().float() @ Wd.t() + mod.scaling * (x.detach().float() @ mod.lora_A.float().t()) @ mod.lora_B.float().t()
    assert ((y.detach().float() - want).norm() / want.norm()).item() <= 1e-2
    assert x.grad is not None and mod.lora_A.grad is not None and mod.lora_B.grad is not None
    assert q.nbytes() < 0.6 * W.numel()
