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
