"""Host-side logic of the package checked on the CPU: shift, advantages and
weights against the oracle (bit-exact group assignment), the synthetic case
generator's invariants, argument validation of the wrappers."""
import hashlib
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import grpo_oracle as O  # noqa: E402

from art_amd import advantage, ops, synthetic  # noqa: E402
from art_amd.train import calculate_attn_bias, shift_tensor  # noqa: E402


def test_shift_matches_oracle_bit_exact():
    g = torch.Generator().manual_seed(0)
    for t, pad in [(torch.randint(0, 1000, (3, 17), generator=g), 0),
                   (torch.rand(2, 9, generator=g) < 0.5, False),
                   (torch.randn(4, 5, generator=g), 0.0)]:
        assert torch.equal(shift_tensor(t, pad), O.shift_tensor(t, pad))


def test_group_advantages_bit_exact_vs_oracle():
    g = np.random.default_rng(0)
    for n_groups, size in [(1, 4), (8, 4), (5, 7), (3, 1)]:
        r = g.random(n_groups * size)
        if n_groups > 1:
            r[size:2 * size] = 0.25  # a zero-variance group
        gid = np.repeat(np.arange(n_groups), size)
        got = advantage.group_advantages(r, gid)
        want = np.array(sum(O.grpo_advantages([list(r[i * size:(i + 1) * size]) for i in range(n_groups)]), []))
        assert got.dtype == np.float64 and np.array_equal(got, want)
        assert np.array_equal(got.astype(np.float32), want.astype(np.float32))
    keep = advantage.keep_mask(advantage.group_advantages([1.0, 1.0, 0.0, 2.0], [0, 0, 1, 1]))
    assert keep.tolist() == [False, False, True, True]


def test_group_assignment_is_by_label_not_position():
    r = [1.0, 5.0, 0.0, 7.0]
    a = advantage.group_advantages(r, [10, 20, 10, 20])
    b = O.grpo_advantages([[1.0, 0.0], [5.0, 7.0]])
    assert [a[0], a[2]] == b[0] and [a[1], a[3]] == b[1]


def test_token_weights_and_advantages_match_oracle():
    case = synthetic.make_grpo_case("t", 5, 1024, 8, 64, 8, 4, (0.2, 0.5), rewards="bernoulli")
    want = O.token_weights(case.assistant_mask, case.traj_id)
    assert torch.allclose(case.weights, want, rtol=1e-6, atol=0)
    assert case.weights[~case.assistant_mask].abs().max().item() == 0.0
    adv = torch.tensor(case.traj_advantages, dtype=torch.float64).to(torch.float32)
    assert torch.equal(case.advantages[0], adv[case.traj_id[0]])


def test_synthetic_case_layout():
    case = synthetic.make_grpo_case("t", 11, 2048, 16, 128, 4, 4, 0.5)
    L = 512
    for j in range(4):
        m = case.assistant_mask[0, j * L:(j + 1) * L]
        assert int(m.sum()) == 256 and not bool(m[0])  # exact density, gap first
        edges = (m[1:] != m[:-1]).sum().item()
        assert edges == 7  # 4 gaps and 4 spans alternating
    assert case.group_of_traj.tolist() == [0, 0, 0, 0]
    # same seed -> same bits
    again = synthetic.make_grpo_case("t", 11, 2048, 16, 128, 4, 4, 0.5)
    for k in ("hidden", "lm_head", "tokens", "assistant_mask", "advantages", "weights", "noise"):
        a, b = getattr(case, k), getattr(again, k)
        assert hashlib.sha256(a.view(torch.uint8).numpy().tobytes() if a.dtype != torch.bfloat16 else a.view(torch.int16).numpy().tobytes()).hexdigest() == \
            hashlib.sha256(b.view(torch.uint8).numpy().tobytes() if b.dtype != torch.bfloat16 else b.view(torch.int16).numpy().tobytes()).hexdigest()
    new = torch.zeros(1, 2048)
    case.finish(new)
    assert torch.isnan(case.logprobs[~case.assistant_mask]).all()
    assert not torch.isnan(case.logprobs[case.assistant_mask]).any()


def test_attn_bias_brute_force():
    g = torch.Generator().manual_seed(2)
    S = 12
    gid = torch.randint(0, 3, (2, S), generator=g)
    pid = torch.randint(0, 3, (2, S), generator=g)
    bias = calculate_attn_bias(2, S, torch.device("cpu"), gid, pid, torch.float32)
    for b in range(2):
        for i in range(S):
            for j in range(S):
                vis = j <= i and (gid[b, i] == gid[b, j] or pid[b, i] == gid[b, j])
                assert bias[b, i, j].item() == (0.0 if vis else float("-inf"))


def test_clip_bounds_python_float_semantics():
    assert ops.clip_bounds(0.2, None) == (1 - 0.2, 1 + 0.2)
    assert ops.clip_bounds(0.2, 0.28) == (1 - 0.2, 1 + 0.28)


def test_wrappers_refuse_cpu_tensors():
    h = torch.zeros(4, 64, dtype=torch.bfloat16)
    w = torch.zeros(8, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.logprob_fwd(h, w, torch.zeros(4, dtype=torch.int64), False, 4)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.transpose(h)


def test_frozen_weight_view_is_stable_until_the_weight_changes():
    """``weight.t()`` is a new view object in every step; the wrapper maps it back to one
    detached bf16 tensor per weight version, so caches keyed by the tensor object hit."""
    from art_amd.train import _as_vh
    w = torch.nn.Parameter(torch.randn(12, 4).to(torch.bfloat16), requires_grad=False)
    a, b = _as_vh(w.t()), _as_vh(w.t())
    assert a is b and a.data_ptr() == w.data_ptr() and a.shape == (12, 4)
    with torch.no_grad():
        w.add_(1)
    c = _as_vh(w.t())
    assert c is not a and torch.equal(c, w)
    w32 = torch.nn.Parameter(torch.randn(12, 4), requires_grad=False)
    d = _as_vh(w32.t())
    assert d is _as_vh(w32.t()) and d.dtype == torch.bfloat16
    plain = torch.randn(4, 12).to(torch.bfloat16)      # an [H, V] tensor that is not such a view
    assert torch.equal(_as_vh(plain), plain.t())
