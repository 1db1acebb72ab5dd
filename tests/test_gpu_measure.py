"""The measurement aids of the library: MFMA-only loops and the plain copy.

The loops have no counterpart in the reference; what is checked is that they do the matrix
work they are credited with: the sum of a wave's accumulators after one round equals the
closed form  sum_s sum_g (sum of the A fragments of K group g) . (sum of the B fragments of g),
evaluated in float64 from the operand indices the kernels document.
"""
import numpy as np
import pytest
import torch

from art_amd import ops

pytestmark = pytest.mark.gpu


def wave_sums_closed_form(operands, shape):
    n = operands.numel()
    x = operands.float().double().numpy()
    if shape == "32x32x16":
        steps, per_step, na, nb, group_shift = 4, 6, 4, 2, 5
    else:
        steps, per_step, na, nb, group_shift = 2, 12, 8, 4, 4
    out = np.zeros(8)
    gid = np.arange(512)

    def frag(s, slot):  # [512 lanes, 8]
        base = ((gid * 24 + s * per_step + slot) * 8) % (n - 8)
        return x[base[:, None] + np.arange(8)[None, :]]

    for s in range(steps):
        a = sum(frag(s, i) for i in range(na))
        b = sum(frag(s, na + j) for j in range(nb))
        for wave in range(8):
            for g in range(64 >> group_shift):
                lanes = [wave * 64 + l for l in range(64) if (l >> group_shift) == g]
                out[wave] += float(a[lanes].sum(0) @ b[lanes].sum(0))
    return out


@pytest.mark.parametrize("shape", ["32x32x16", "16x16x32"])
def test_mfma_loop_does_the_work_it_is_credited_with(artk_lib, gpu, shape):
    print(f"mfma_loop {shape}", flush=True)
    g = torch.Generator().manual_seed(11)
    operands = torch.randn(1 << 14, generator=g).to(torch.bfloat16)
    sink = torch.zeros(512, dtype=torch.float32, device=gpu)
    flop = ops.mfma_loop(operands.to(gpu), 1, 1, sink, shape=shape)
    assert flop == 8 * 32 * 32768.0
    got = sink.cpu().double().view(8, 64).sum(1).numpy()
    want = wave_sums_closed_form(operands, shape)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-3 * scale + 1e-2, (got, want)
    sink3 = torch.zeros_like(sink)
    ops.mfma_loop(operands.to(gpu), 3, 1, sink3, shape=shape)
    got3 = sink3.cpu().double().view(8, 64).sum(1).numpy()
    assert np.abs(got3 - 3 * want).max() <= 3e-3 * scale + 3e-2


def test_mfma_loop_rejects_bad_arguments(artk_lib, gpu):
    operands = torch.zeros(4096, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        ops.mfma_loop(operands, 1, 1, shape="4x4x4")
    with pytest.raises((ValueError, RuntimeError)):
        ops.mfma_loop(operands[:1024], 1, 1)


def test_stream_copy_is_a_copy(artk_lib, gpu):
    src = torch.arange(1 << 20, dtype=torch.int32, device=gpu)
    dst = torch.zeros_like(src)
    assert ops.stream_copy(src, dst) == src.numel() * 4
    assert torch.equal(src, dst)


@pytest.mark.parametrize("waves,kind,rpd", [(8, 0, 0), (4, 1, 2), (8, 2, 3)])
def test_lds_probe_reports_a_plausible_rate(artk_lib, gpu, waves, kind, rpd):
    print(f"lds_probe waves={waves} kind={kind} rpd={rpd}", flush=True)
    r = ops.lds_probe(waves, kind, rpd, 200, 4, gpu)
    # a CU cannot read more than a few hundred bytes per clock from LDS, nor fewer than a few
    assert 8.0 < r["read_B_per_clk"] < 1024.0, r
    assert (r["dma_write_B_per_clk"] > 0) == (rpd > 0)
    with pytest.raises(ValueError):
        ops.lds_probe(3, 0, 0, 1, 1, gpu)


@pytest.mark.parametrize("loop,group", [(0, 8), (1, 4), (2, 8), (2, 4), (3, 4), (4, 8), (4, 4), (5, 8), (5, 4)])
def test_gemm_loop_probe_computes_the_product(artk_lib, gpu, loop, group):
    """Without ablation switches every loop variant of the probe is a correct GEMM (fp32 matmul of the
    bf16 inputs, bf16 rounding of the result); with a switch set it still runs to completion."""
    print(f"gemm_loop_probe loop={loop} group={group}", flush=True)
    g = torch.Generator().manual_seed(3 + loop)
    M, N, K = 2304, 2048, 320
    p = torch.randn(M, K, generator=g).to(torch.bfloat16).to(gpu)
    q = torch.randn(N, K, generator=g).to(torch.bfloat16).to(gpu)
    cyc = torch.zeros(2 * torch.cuda.get_device_properties(gpu).multi_processor_count, dtype=torch.int64, device=gpu)
    out = ops.gemm_loop_probe(p, q, loop=loop, group=group, cycles=cyc)
    ref = q.float() @ p.float().t()
    rel = ((out.float() - ref).norm() / ref.norm()).item()
    assert rel < 4e-3, rel
    assert int(cyc[0]) > 0 and int(cyc[1]) > 0
    if loop in (2, 3):
        for ablate in (1, 2, 4, 7):
            ops.gemm_loop_probe(p, q, loop=loop, ablate=ablate, group=group, same_tile=True)
        torch.cuda.synchronize()
    if loop == 5:  # its second variant is a correct GEMM too
        out1 = ops.gemm_loop_probe(p, q, loop=5, ablate=1, group=group)
        assert ((out1.float() - ref).norm() / ref.norm()).item() < 4e-3
    with pytest.raises(ValueError):
        ops.gemm_loop_probe(p, q, loop=1, ablate=1)
