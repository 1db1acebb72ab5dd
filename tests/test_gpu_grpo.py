"""GPU parity of the GRPO logprob / loss path against the CPU oracle.

Tolerances (fp32 oracle on the bf16-valued inputs): per-token logprob <= 2e-3
abs, loss <= 1e-3 rel, d_hidden <= 1e-2 rel-L2; indices and masks bit-exact
(an off-by-one shift or a wrong gather index shows up as O(1) logprob errors).
"""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import grpo_oracle  # noqa: E402

from art_amd import ops, synthetic  # noqa: E402
from art_amd.train import _calculate_logprobs, fused_grpo_loss, grpo_loss, shift_tensor  # noqa: E402

pytestmark = pytest.mark.gpu

LP_TOL, LOSS_TOL, GRAD_TOL = 2e-3, 1e-3, 1e-2


def rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def oracle_case(case, chunk):
    new = grpo_oracle.calculate_logprobs(case.lm_head.float().t(), case.hidden.float(),
                                         grpo_oracle.shift_tensor(case.tokens, 0), chunk)
    case.finish(new)
    return grpo_oracle.loss_and_grad(case.hidden, case.lm_head, case.tokens, case.logprobs,
                                     case.advantages, case.assistant_mask, case.weights,
                                     chunk_size=chunk)


@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 768, 256), (264, 300, 128), (8, 1, 64),
                                   (1024, 512, 1024), (5004, 4100, 128), (6152, 3330, 64)])
def test_gemm_nt_matches_fp32_matmul(artk_lib, gpu, M, N, K):
    """The last two shapes have more tiles than the part has CUs (each work-group walks several) and ragged
    edges on both sides (rows past the end of either operand read as zeros and are never stored; M % 8 != 0
    takes the 8-byte store path)."""
    print(f"gemm_nt M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M * 7 + N)
    p = torch.randn(M, K, generator=g).to(torch.bfloat16)
    q = torch.randn(N, K, generator=g).to(torch.bfloat16)
    ref = q.float() @ p.float().t()
    out = ops.gemm_nt(p.to(gpu), q.to(gpu), out_f32=True).cpu()
    assert rel_l2(out, ref) < 1e-5
    out16 = ops.gemm_nt(p.to(gpu), q.to(gpu), out_f32=False).cpu().float()
    assert rel_l2(out16, ref) < 4e-3


def test_transpose(artk_lib, gpu):
    x = torch.randn(200, 328).to(torch.bfloat16)
    assert torch.equal(ops.transpose(x.to(gpu)).cpu(), x.t().contiguous())


@pytest.mark.parametrize("T,H,V,B", [(512, 256, 8192, 1), (384, 192, 8000, 2), (256, 64, 1000, 1),
                                     (40, 128, 50008, 1)])
def test_logprob_fwd_matches_oracle(artk_lib, gpu, T, H, V, B):
    print(f"logprob_fwd T={T} H={H} V={V} B={B}", flush=True)
    g = torch.Generator().manual_seed(T + V)
    hidden = torch.randn(B, T // B, H, generator=g).to(torch.bfloat16)
    lm_head = (0.05 * torch.randn(V, H, generator=g)).to(torch.bfloat16)
    tokens = torch.randint(0, V, (B, T // B), generator=g)
    tokens[0, 0] = V - 1  # last vocab row, inside the ragged tile
    tokens[0, 1] = 0
    nxt = grpo_oracle.shift_tensor(tokens, 0)
    ref = grpo_oracle.calculate_logprobs(lm_head.float().t(), hidden.float(), nxt, T // B)
    # un-shifted ids + in-kernel shift
    lp, lse = ops.logprob_fwd(hidden.view(T, H).to(gpu), lm_head.to(gpu), tokens.view(T).to(gpu), True,
                              T // B)
    assert (lp.cpu().view(B, -1) - ref).abs().max().item() <= LP_TOL
    # pre-shifted ids, no shift: the drop-in signature
    lp2 = _calculate_logprobs(lm_head.to(gpu).t(), hidden.to(gpu), nxt.to(gpu), T // B)
    assert torch.equal(lp2.view(-1), lp)
    ref_lse = torch.logsumexp(hidden.float().view(T, H) @ lm_head.float().t(), -1)
    assert (lse.cpu() - ref_lse).abs().max().item() <= 1e-4


def test_logprob_invalid_id_is_nan(artk_lib, gpu):
    hidden = torch.randn(256, 64).to(torch.bfloat16).to(gpu)
    lm_head = torch.randn(512, 64).to(torch.bfloat16).to(gpu)
    ids = torch.zeros(256, dtype=torch.int64)
    ids[5] = -100
    ids[6] = 512
    lp, _ = ops.logprob_fwd(hidden, lm_head, ids.to(gpu), False, 256)
    lp = lp.cpu()
    assert torch.isnan(lp[5]) and torch.isnan(lp[6]) and not torch.isnan(lp[7])


@pytest.mark.parametrize("T,H,V,n_traj,chunk_tokens", [(512, 256, 8192, 4, 4096), (768, 192, 8000, 4, 256),
                                                       (1024, 128, 4096, 8, 384), (1000, 192, 8000, 4, 0),
                                                       (520, 64, 4160, 4, 200)])
def test_fused_matches_oracle(artk_lib, gpu, T, H, V, n_traj, chunk_tokens):
    print(f"fused T={T} H={H} V={V} chunk={chunk_tokens}", flush=True)
    case = synthetic.make_grpo_case("t", T + H, T, H, V, n_traj, 4, 0.5)
    ref = oracle_case(case, T // 2)
    hidden = case.hidden.to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(
        hidden, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu),
        case.advantages.to(gpu), case.assistant_mask.to(gpu), case.weights.to(gpu),
        chunk_tokens=chunk_tokens)
    loss.backward()
    assert (logprob.cpu() - ref["logprobs"]).abs().max().item() <= LP_TOL
    assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
    assert metrics["mask_count"].item() == grpo_oracle.shift_tensor(case.assistant_mask, False).sum().item()
    assert rel_l2(hidden.grad.float().cpu(), ref["d_hidden"]) <= GRAD_TOL
    # rows whose shifted mask is 0 get exactly zero gradient
    m = grpo_oracle.shift_tensor(case.assistant_mask, False)[0]
    assert hidden.grad[0][~m.to(gpu)].abs().max().item() == 0.0


def test_fused_wide_logit_range(artk_lib, gpu):
    """Peaked distributions: logits spread over +-35 nats, targets up to ~65 nats under their row's maximum.
    The backward works on exp(logit - target logit) in bf16, which has to hold over that range."""
    T, H, V = 512, 256, 8192
    case = synthetic.make_grpo_case("w", 31, T, H, V, 4, 4, 0.5)
    case.hidden = (case.hidden.float() * 25.0).to(torch.bfloat16)
    ref = oracle_case(case, T)
    logits = case.hidden[0].float() @ case.lm_head.float().t()
    nxt = grpo_oracle.shift_tensor(case.tokens, 0)[0]
    gap = logits.max(-1).values - logits.gather(1, nxt.view(-1, 1)).squeeze(1)
    assert 40.0 < gap.max().item() < 80.0
    hidden = case.hidden.to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(
        hidden, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu),
        case.advantages.to(gpu), case.assistant_mask.to(gpu), case.weights.to(gpu))
    loss.backward()
    assert (logprob.cpu() - ref["logprobs"]).abs().max().item() <= 2e-3 * 25
    assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item()) + 2e-6
    assert torch.isfinite(hidden.grad).all()
    assert rel_l2(hidden.grad.float().cpu(), ref["d_hidden"]) <= GRAD_TOL


def test_fused_target_far_under_the_maximum_is_dropped_and_counted(artk_lib, gpu):
    """A sampled token whose logit lies 95 nats under its row's largest one (probability below
    e^-80: it cannot have been sampled) would overflow the exponential stash.  That row's d_hidden
    is written as zeros and counted in metrics["dropped_rows"]; its logprob and the loss stay exact
    and finite, every other row is unaffected, nothing in d_hidden is inf or NaN."""
    T, H, V = 256, 64, 1024
    hidden = torch.zeros(1, T, H, dtype=torch.bfloat16)
    hidden[0, :, 0] = 1.0
    lm_head = torch.zeros(V, H, dtype=torch.bfloat16)
    lm_head[:, 0] = -20.0
    lm_head[7, 0] = 50.0                      # one dominant logit
    lm_head[9, 0] = -45.0                     # 95 nats under it
    lm_head[:, 1] = (torch.arange(V) % 5).to(torch.bfloat16)   # (unused direction: hidden[.., 1] = 0)
    tokens = torch.full((1, T), 7, dtype=torch.int64)
    tokens[0, 101] = 9                        # position 100's target
    old = torch.zeros(1, T)
    old[0, 101] = -95.0                       # ratio 1: the row has a non-zero coefficient
    adv = torch.ones(1, T)
    mask = torch.ones(1, T, dtype=torch.bool)
    w = torch.ones(1, T)
    for skip in (False, True):
        h = hidden.to(gpu).requires_grad_(True)
        loss, metrics, logprob = fused_grpo_loss(h, lm_head.to(gpu), tokens.to(gpu), old.to(gpu), adv.to(gpu),
                                                 mask.to(gpu), w.to(gpu), skip_inactive=skip)
        loss.backward()
        g = h.grad[0].float().cpu()
        assert abs(logprob[0, 100].item() + 95.0) < 1e-3
        assert torch.isfinite(loss).item() and torch.isfinite(g).all()
        assert metrics["dropped_rows"].item() == 1.0
        assert (g[100] == 0).all()
        # every other row against the oracle (their targets carry all of the probability, so the
        # rows are tiny: an absolute bound)
        ref = grpo_oracle.loss_and_grad(hidden, lm_head, tokens, old, adv, mask, w, 0.2, 0.2, chunk_size=T)
        want = ref["d_hidden"][0]
        others = torch.cat([torch.arange(100), torch.arange(101, T)])
        assert (g[others] - want[others]).abs().max().item() <= 1e-6
        assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item()) + 2e-6


def test_fused_no_grad_runs_the_forward_half_only(artk_lib, gpu):
    """Under torch.no_grad() (an evaluation pass) the loss comes from the forward kernels alone
    and equals the training pass's loss and logprobs up to fp32 rounding (the training pass sums a
    stashed row's exponentials against the row's target logit, the evaluation pass against the
    running maximum)."""
    T, H, V = 512, 128, 4096
    case = synthetic.make_grpo_case("t", 98, T, H, V, 4, 4, 0.5)
    oracle_case(case, 256)   # fills in the old logprobs
    args = (case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu), case.advantages.to(gpu),
            case.assistant_mask.to(gpu), case.weights.to(gpu))
    h = case.hidden.to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(h, *args)
    from art_amd import ops
    ops.profile_enable(True)
    with torch.no_grad():
        loss2, metrics2, logprob2 = fused_grpo_loss(h, *args)
    torch.cuda.synchronize()
    _, n_bwd = ops.profile_collect(ops.PROF_DHIDDEN_GEMM)
    _, n_fwd = ops.profile_collect(ops.PROF_LMHEAD_FWD)
    ops.profile_enable(False)
    assert n_fwd >= 1 and n_bwd == 0
    # (the loss is a mean of signed terms of order 1e-2 that nearly cancel)
    assert abs(loss2.item() - loss.item()) <= 1e-4 * abs(loss.item()) + 1e-7
    assert torch.equal(torch.isnan(logprob2), torch.isnan(logprob))
    ok = ~torch.isnan(logprob)
    assert (logprob2[ok] - logprob[ok]).abs().max().item() <= 1e-5
    assert abs(metrics2["policy_loss"].item() - metrics["policy_loss"].item()) <= (
        1e-4 * abs(metrics["policy_loss"].item()) + 1e-7)
    assert metrics2["dropped_rows"].item() == 0.0
    assert not loss2.requires_grad


def test_unfused_autograd_matches_oracle(artk_lib, gpu):
    """_calculate_logprobs + grpo_loss composed through torch autograd (the
    reference's call structure) against the oracle, with KL."""
    T, H, V = 512, 128, 4096
    case = synthetic.make_grpo_case("t", 99, T, H, V, 4, 4, 0.5)
    oracle_case(case, 256)
    g = torch.Generator().manual_seed(5)
    ref_lp = case.logprobs.nan_to_num(-8.0) + 0.1 * torch.randn(1, T, generator=g)
    ref_lp = grpo_oracle.shift_tensor(ref_lp, 0.0)
    beta = 0.05
    ref = grpo_oracle.loss_and_grad(case.hidden, case.lm_head, case.tokens, case.logprobs,
                                    case.advantages, case.assistant_mask, case.weights,
                                    chunk_size=256, ref_logprobs=ref_lp, beta=beta)
    hidden = case.hidden.to(gpu).requires_grad_(True)
    nxt = shift_tensor(case.tokens.to(gpu), 0)
    new = _calculate_logprobs(case.lm_head.to(gpu).t(), hidden, nxt, 256)
    loss, metrics = grpo_loss(
        new, shift_tensor(case.logprobs.to(gpu), 0.0), shift_tensor(case.advantages.to(gpu), 0.0),
        shift_tensor(case.assistant_mask.to(gpu), False), shift_tensor(case.weights.to(gpu), 0.0),
        ref_logprobs=ref_lp.to(gpu), beta=beta)
    loss.backward()
    assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
    assert abs(metrics["kl_div"].item() - ref["kl"].item()) <= LOSS_TOL * abs(ref["kl"].item())
    assert rel_l2(hidden.grad.float().cpu(), ref["d_hidden"]) <= GRAD_TOL
    # fused path with KL gives the same numbers
    h2 = case.hidden.to(gpu).requires_grad_(True)
    loss2, m2, _ = fused_grpo_loss(h2, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu),
                                   case.advantages.to(gpu), case.assistant_mask.to(gpu),
                                   case.weights.to(gpu), ref_logprobs=ref_lp.to(gpu), beta=beta)
    loss2.backward()
    assert abs(loss2.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
    assert rel_l2(h2.grad.float().cpu(), ref["d_hidden"]) <= GRAD_TOL


def test_fused_is_deterministic(artk_lib, gpu):
    case = synthetic.make_grpo_case("t", 3, 512, 128, 4096, 4, 4, 0.5)
    oracle_case(case, 256)
    dev = case.to(gpu)
    outs = []
    for _ in range(2):
        s, lp, dh = ops.grpo_fused(dev.hidden.view(512, 128), dev.lm_head, ops.transpose(dev.lm_head),
                                   dev.tokens.view(-1), dev.logprobs.view(-1), dev.advantages.view(-1),
                                   dev.assistant_mask.view(-1), dev.weights.view(-1), None, 512, 0.8,
                                   1.2, 0.0)
        outs.append((s.clone(), lp.clone(), dh.clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("density", [0.0, 1.0])
def test_fused_all_or_no_rows_active(artk_lib, gpu, density):
    """Edge cases of the active-row compaction: empty mask (zero loss, zero
    gradient, no GEMM work) and a mask covering every position."""
    T, H, V = 512, 128, 4096
    case = synthetic.make_grpo_case("t", 17, T, H, V, 4, 4, 0.5)
    case.assistant_mask = torch.full_like(case.assistant_mask, bool(density))
    from art_amd.advantage import token_weights
    case.weights = token_weights(case.assistant_mask, case.traj_id) if density else torch.zeros_like(case.weights)
    ref = oracle_case(case, 256)
    hidden = case.hidden.to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(
        hidden, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu),
        case.advantages.to(gpu), case.assistant_mask.to(gpu), case.weights.to(gpu), chunk_tokens=256)
    loss.backward()
    assert (logprob.cpu() - ref["logprobs"]).abs().max().item() <= LP_TOL
    if density == 0.0:
        assert loss.item() == 0.0 and hidden.grad.abs().max().item() == 0.0
        assert metrics["mask_count"].item() == 0
    else:
        assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
        assert rel_l2(hidden.grad.float().cpu(), ref["d_hidden"]) <= GRAD_TOL
        assert metrics["mask_count"].item() == T - 1  # the last position's mask shifts out


@pytest.mark.parametrize("T,H,V,n_traj,chunk_tokens,density,beta",
                         [(512, 256, 8192, 4, 4096, 0.5, 0.0), (1024, 128, 4096, 8, 256, 0.3, 0.0),
                          (768, 192, 8000, 4, 256, 0.5, 0.05), (512, 128, 4096, 4, 256, 0.0, 0.0),
                          (512, 128, 4096, 4, 256, 1.0, 0.0)])
def test_fused_skip_inactive(artk_lib, gpu, T, H, V, n_traj, chunk_tokens, density, beta):
    """Projecting only the positions that can contribute gives the oracle's loss
    and gradient, the dense mode's loss bit for bit, and NaN logprobs exactly at
    the skipped positions."""
    print(f"fused skip T={T} H={H} V={V} chunk={chunk_tokens} density={density} beta={beta}", flush=True)
    case = synthetic.make_grpo_case("t", T + H + 1, T, H, V, n_traj, 4, 0.5)
    if density in (0.0, 1.0):
        from art_amd.advantage import token_weights
        case.assistant_mask = torch.full_like(case.assistant_mask, bool(density))
        case.weights = (token_weights(case.assistant_mask, case.traj_id) if density
                        else torch.zeros_like(case.weights))
    oracle_case(case, T // 2)
    ref_lp = None
    if beta > 0:
        g = torch.Generator().manual_seed(11)
        ref_lp = grpo_oracle.shift_tensor(
            case.logprobs.nan_to_num(-8.0) + 0.1 * torch.randn(1, T, generator=g), 0.0)
    ref = grpo_oracle.loss_and_grad(case.hidden, case.lm_head, case.tokens, case.logprobs,
                                    case.advantages, case.assistant_mask, case.weights,
                                    chunk_size=T // 2, ref_logprobs=ref_lp, beta=beta)
    res = {}
    for skip in (False, True):
        hidden = case.hidden.to(gpu).requires_grad_(True)
        loss, metrics, logprob = fused_grpo_loss(
            hidden, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu),
            case.advantages.to(gpu), case.assistant_mask.to(gpu), case.weights.to(gpu),
            ref_logprobs=None if ref_lp is None else ref_lp.to(gpu), beta=beta,
            chunk_tokens=chunk_tokens, skip_inactive=skip)
        loss.backward()
        res[skip] = (loss.detach().cpu(), metrics, logprob.cpu(), hidden.grad.float().cpu())
    loss, metrics, logprob, grad = res[True]
    assert torch.equal(loss, res[False][0])
    assert torch.equal(metrics["policy_loss"].cpu(), res[False][1]["policy_loss"].cpu())
    assert torch.equal(metrics["kl_div"].cpu(), res[False][1]["kl_div"].cpu())
    assert metrics["mask_count"].item() == res[False][1]["mask_count"].item()
    # which positions are evaluated
    sh = lambda t, fill: grpo_oracle.shift_tensor(t, fill)
    want = sh(case.assistant_mask, False) & (sh(case.weights, 0.0) != 0)
    if beta == 0:
        want &= sh(case.advantages, 0.0) != 0
    assert torch.equal(~torch.isnan(logprob), want)
    assert torch.equal(logprob[want], res[False][2][want])
    if density == 0.0:
        assert loss.item() == 0.0 and grad.abs().max().item() == 0.0
        return
    assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
    assert rel_l2(grad, ref["d_hidden"]) <= GRAD_TOL
    assert rel_l2(grad, res[False][3]) <= 2e-3  # bf16 rounding of differently ordered fp32 sums
    assert grad[0][~want[0]].abs().max().item() == 0.0


def test_config1_full_size(artk_lib, gpu):
    """Benchmark config 1 (Qwen2.5-0.5B shape) at full size against the oracle."""
    print("config1 full size", flush=True)
    case = synthetic.config1()
    ref = oracle_case(case, 1024)
    hidden = case.hidden.to(gpu).requires_grad_(True)
    loss, metrics, logprob = fused_grpo_loss(
        hidden, case.lm_head.to(gpu), case.tokens.to(gpu), case.logprobs.to(gpu),
        case.advantages.to(gpu), case.assistant_mask.to(gpu), case.weights.to(gpu))
    loss.backward()
    assert (logprob.cpu() - ref["logprobs"]).abs().max().item() <= LP_TOL
    assert abs(loss.item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
    assert rel_l2(hidden.grad.float().cpu(), ref["d_hidden"]) <= GRAD_TOL


# ---------------------------------------------------------------------------------
# Full-size configurations (benchmark configs 3 and 4): the CPU oracle cannot run the
# whole case in seconds, so parity is checked on windows of positions (every
# position's logprob and d_hidden row depend on the rest of the batch only through
# the scalar mask count) and through size-independent properties.
# ---------------------------------------------------------------------------------
def window_oracle(case, start, length, mask_count_full):
    """Oracle logprobs and d_hidden rows for positions [start, start+length-1) of a
    full-size case, evaluated on the window alone and rescaled to the batch's denominator."""
    sl = slice(start, start + length)
    cut = lambda t: t[:, sl].contiguous()
    out = grpo_oracle.loss_and_grad(cut(case.hidden), case.lm_head, cut(case.tokens), cut(case.logprobs),
                                    cut(case.advantages), cut(case.assistant_mask), cut(case.weights),
                                    chunk_size=length)
    m_win = grpo_oracle.shift_tensor(cut(case.assistant_mask), False).sum().item()
    scale = (m_win + 1e-6) / (mask_count_full + 1e-6)
    return out["logprobs"][0, :-1], out["d_hidden"][0, :-1] * scale


def run_full_size(case, gpu, chunk_tokens):
    T, H = case.hidden.shape[1], case.hidden.shape[2]
    dev = case.to(gpu)
    lm_head_t = ops.transpose(dev.lm_head)
    new, _ = ops.logprob_fwd(dev.hidden.view(T, H), dev.lm_head, dev.tokens.view(T), True, T)
    case.finish(new.cpu())
    old = case.logprobs.view(T).to(gpu)
    args = (dev.hidden.view(T, H), dev.lm_head, lm_head_t, dev.tokens.view(T), old, dev.advantages.view(T),
            dev.assistant_mask.view(T), dev.weights.view(T), None, T, 0.8, 1.2, 0.0)
    s, lp, dh = ops.grpo_fused(*args, chunk_tokens)
    return args, s, lp, dh, new


@pytest.mark.parametrize("name", ["c3", "c4"])
def test_full_size_windows_and_properties(artk_lib, gpu, name):
    print(f"full size {name}", flush=True)
    case = synthetic.config3() if name == "c3" else synthetic.config4()
    T, H = case.hidden.shape[1], case.hidden.shape[2]
    args, s, lp, dh, new = run_full_size(case, gpu, 4096)
    count = grpo_oracle.shift_tensor(case.assistant_mask, False).sum().item()
    assert s[3].item() == count                       # integer mask count, bit-exact
    assert same_logprobs(lp, new)                      # fused forward == forward-only kernel
    # windows: start of the row, a trajectory boundary, the end of the row
    L = T // (32 if name == "c3" else 16)
    for start in (0, 3 * L - 40, T - 96):
        ref_lp, ref_dh = window_oracle(case, start, 96, count)
        got_lp = lp[start:start + 95].cpu()
        got_dh = dh[start:start + 95].float().cpu()
        assert (got_lp - ref_lp).abs().max().item() <= LP_TOL
        if ref_dh.abs().max().item() == 0.0:  # a window inside a zero-advantage group
            assert got_dh.abs().max().item() == 0.0
        else:
            assert rel_l2(got_dh, ref_dh) <= GRAD_TOL
    # rows with a zero coefficient (mask off, or zero advantage) are exactly zero
    m = grpo_oracle.shift_tensor(case.assistant_mask, False)[0]
    a = grpo_oracle.shift_tensor(case.advantages, 0.0)[0]
    dead = (~m) | (a == 0)
    assert dh[dead.to(gpu)].abs().max().item() == 0.0
    # the remaining rows carry gradient unless the ratio was clipped (coefficient exactly 0)
    nonzero = dh[(~dead).to(gpu)].float().abs().amax(dim=1) > 0
    assert nonzero.float().mean().item() > 0.5
    if name == "c4":
        assert (a[m] == 0).any(), "config 4 must contain zero-variance groups"
    # chunk-size invariance: forward bit-identical, loss and gradient within tolerance
    s2, lp2, dh2 = ops.grpo_fused(*args, 2048)
    assert torch.equal(lp2, lp)
    assert abs(s2[0].item() - s[0].item()) <= 1e-6 * abs(s[0].item())
    assert rel_l2(dh2.float(), dh.float()) <= 1e-3
    # run-to-run determinism
    s3, lp3, dh3 = ops.grpo_fused(*args, 4096)
    assert torch.equal(s3, s) and torch.equal(dh3, dh)
    # loss scalar against the oracle's loss body fed with the kernel's logprobs
    loss_ref, _, _ = grpo_oracle.grpo_loss(
        lp.cpu().view(1, T), grpo_oracle.shift_tensor(case.logprobs, 0.0),
        grpo_oracle.shift_tensor(case.advantages, 0.0),
        grpo_oracle.shift_tensor(case.assistant_mask, False).float(),
        grpo_oracle.shift_tensor(case.weights, 0.0))
    assert abs(s[0].item() - loss_ref.item()) <= LOSS_TOL * abs(loss_ref.item())
    # skipping the positions that cannot contribute: same loss bit for bit, same gradient
    s4, lp4, dh4 = ops.grpo_fused(*args, 4096, skip_inactive=True)
    assert torch.equal(s4, s)
    assert torch.equal(torch.isnan(lp4), dead.to(gpu))
    assert torch.equal(lp4[(~dead).to(gpu)], lp[(~dead).to(gpu)])
    assert rel_l2(dh4.float(), dh.float()) <= 2e-3
    assert dh4[dead.to(gpu)].abs().max().item() == 0.0


def same_logprobs(a, b, tol=2e-5):
    """The fused step and the forward-only entry point agree up to fp32 rounding: the fused step sums
    a stashed row's exponentials against the row's target logit, the forward-only kernel against the
    running maximum.  NaN (no target) in the same places."""
    if not torch.equal(torch.isnan(a), torch.isnan(b)):
        return False
    ok = ~torch.isnan(a)
    return (a[ok] - b[ok]).abs().max().item() <= tol


def chunk_bounds(T, V):
    """First positions of the chunks the library forms by itself (chunk_tokens = 0): about 6000
    positions per chunk, the batch's 256-position tiles spread evenly over the chunks."""
    cap = max(((1 << 30) - 1) // V // 256 * 256, 256)
    want = min(cap, 6144)
    n = -(-T // want)
    tc = min(-(-(-(-T // n)) // 256) * 256, cap, T)
    nchunks, tiles = -(-T // tc), -(-T // 256)
    base, extra = divmod(tiles, nchunks)
    bounds, t0 = [], 0
    for c in range(nchunks):
        bounds.append(t0)
        t0 += (base + (1 if c < extra else 0)) * 256
    return bounds


@pytest.mark.parametrize("name", ["c3", "c4"])
def test_full_size_library_chunking_and_independent_loss(artk_lib, gpu, name):
    """Benchmark configs 3 and 4 with the chunking the library picks by itself (uneven chunks:
    22 + 21 + 21 tiles at the 7B shape): windows across a chunk boundary, inside the last chunk
    and at the end of the batch against the CPU oracle; then the WHOLE batch (every logprob, the
    loss, every d_hidden row) against the oracle's own code evaluated in fp32 by torch on the GPU,
    which shares nothing with the kernels."""
    print(f"full size, library chunking {name}", flush=True)
    case = synthetic.config3() if name == "c3" else synthetic.config4()
    T, H = case.hidden.shape[1], case.hidden.shape[2]
    V = case.lm_head.shape[0]
    args, s, lp, dh, new = run_full_size(case, gpu, 0)
    count = grpo_oracle.shift_tensor(case.assistant_mask, False).sum().item()
    assert s[3].item() == count
    assert same_logprobs(lp, new)
    bounds = chunk_bounds(T, V)
    assert len(bounds) >= 3 and bounds[1] - bounds[0] != bounds[-1] - bounds[-2]  # uneven chunks
    starts = (bounds[1] - 48, bounds[-1] - 48, bounds[-1] + 700, T - 96)
    for start in starts:
        ref_lp, ref_dh = window_oracle(case, start, 96, count)
        got_lp = lp[start:start + 95].cpu()
        got_dh = dh[start:start + 95].float().cpu()
        assert (got_lp - ref_lp).abs().max().item() <= LP_TOL, start
        if ref_dh.abs().max().item() == 0.0:
            assert got_dh.abs().max().item() == 0.0
        else:
            assert rel_l2(got_dh, ref_dh) <= GRAD_TOL, start
    # same batch with even chunks of 4096: forward identical, gradient to rounding
    s2, lp2, dh2 = ops.grpo_fused(*args, 4096)
    assert torch.equal(lp2, lp)
    assert rel_l2(dh2.float(), dh.float()) <= 1e-3
    del dh2
    # whole batch against the oracle's code in fp32 on the GPU (rocBLAS fp32 matmul, torch
    # logsumexp / gather / autograd): an evaluation independent of the kernels at full size
    g = lambda t: t.to(gpu)
    ref = grpo_oracle.loss_and_grad(g(case.hidden), g(case.lm_head), g(case.tokens), g(case.logprobs),
                                    g(case.advantages), g(case.assistant_mask), g(case.weights), chunk_size=1024)
    assert (lp - ref["logprobs"][0]).abs().max().item() <= LP_TOL
    assert abs(s[0].item() - ref["loss"].item()) <= LOSS_TOL * abs(ref["loss"].item())
    assert abs(s[1].item() - ref["policy_loss"].item()) <= LOSS_TOL * abs(ref["policy_loss"].item())
    assert rel_l2(dh.float(), ref["d_hidden"][0]) <= GRAD_TOL
    # row by row, so that a few wrong rows cannot hide in the global norm
    num = (dh.float() - ref["d_hidden"][0]).norm(dim=1)
    den = ref["d_hidden"][0].norm(dim=1)
    live = den > 0
    assert (num[live] / den[live]).max().item() <= 3e-2
    assert dh[~live].abs().max().item() == 0.0
