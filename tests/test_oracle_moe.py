"""Pins of oracle/moe_oracle.py: brute force on tiny inputs, library routines and
invariants of the permutation."""
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import moe_oracle as M  # noqa: E402


def test_route_brute_force_with_ties():
    logits = torch.tensor([[0.0, 2.0, 2.0, -1.0], [1.0, 1.0, 1.0, 1.0], [3.0, 0.0, 0.5, 4.0]])
    r = M.route(logits, 2)
    assert r["topk_idx"].tolist() == [[1, 2], [0, 1], [3, 0]]  # ties -> lower index
    p = torch.softmax(logits, -1)
    for t in range(3):
        chosen = [p[t, e].item() for e in r["topk_idx"][t].tolist()]
        want = [c / sum(chosen) for c in chosen]
        assert all(abs(a - b) < 1e-6 for a, b in zip(r["topk_w"][t].tolist(), want))
    # flat keys (token-major): [1,2, 0,1, 3,0] -> stable sort: 0@2, 0@5, 1@0, 1@3, 2@1, 3@4
    assert r["perm"].tolist() == [2, 5, 0, 3, 1, 4]
    assert r["offsets"].tolist() == [0, 2, 4, 5, 6]
    assert r["row_token"].tolist() == [1, 2, 0, 1, 0, 2]


def test_route_nan_and_masked_rows():
    """NaN counts as -inf; ties among -inf go to the lower index; weights of -inf experts are 0,
    and a row without any finite logit has all weights 0 (hand-computed)."""
    ninf, nan = float("-inf"), float("nan")
    logits = torch.tensor([[nan, nan, nan, nan],          # nothing finite: experts 0, 1
                           [ninf, 2.0, ninf, ninf],       # one finite: expert 1, then 0
                           [1.0, nan, 1.0, 3.0],          # 3, then the tie 0 < 2
                           [ninf, ninf, 0.0, 0.0]])       # 2, 3
    r = M.route(logits, 2)
    assert r["topk_idx"].tolist() == [[0, 1], [1, 0], [3, 0], [2, 3]]
    e2 = 1.0 / (1.0 + torch.exp(torch.tensor(-2.0)).item())
    want = [[0.0, 0.0], [1.0, 0.0], [e2, 1.0 - e2], [0.5, 0.5]]
    assert torch.allclose(r["topk_w"], torch.tensor(want), atol=1e-6)
    assert 0 <= int(r["topk_idx"].min()) and int(r["topk_idx"].max()) < 4
    assert sorted(r["perm"].tolist()) == list(range(8))


def test_route_matches_topk_and_invariants():
    g = torch.Generator().manual_seed(0)
    T, E, k = 300, 16, 4
    logits = torch.randn(T, E, generator=g)
    r = M.route(logits, k)
    want = torch.topk(torch.softmax(logits, -1), k, dim=-1).indices  # no ties in random data
    assert torch.equal(r["topk_idx"], want)
    assert torch.allclose(r["topk_w"].sum(-1), torch.ones(T))
    perm = r["perm"]
    assert sorted(perm.tolist()) == list(range(T * k))
    keys = r["topk_idx"].reshape(-1)[perm]
    assert torch.equal(keys, keys.sort().values)
    for e in range(E):  # rows of one expert keep the token-major order
        seg = perm[r["offsets"][e]:r["offsets"][e + 1]]
        assert torch.equal(seg, seg.sort().values)
    assert torch.equal(r["inv_perm"][perm], torch.arange(T * k))


def test_grouped_lora_explicit():
    g = torch.Generator().manual_seed(1)
    E, n_in, n_out, r = 3, 4, 5, 2
    x = torch.randn(7, n_in, generator=g, dtype=torch.float64)
    W = torch.randn(E, n_out, n_in, generator=g, dtype=torch.float64)
    A = torch.randn(E, r, n_in, generator=g, dtype=torch.float64)
    B = torch.randn(E, n_out, r, generator=g, dtype=torch.float64)
    offsets = torch.tensor([0, 3, 3, 7])  # expert 1 has no rows
    y = M.grouped_lora(x, W, A, B, 2.0, offsets)
    for i in range(7):
        e = 0 if i < 3 else 2
        want = W[e] @ x[i] + 2.0 * B[e] @ (A[e] @ x[i])
        assert torch.allclose(y[i], want, atol=1e-12)
    up = torch.randn(7, n_out, generator=g, dtype=torch.float64)
    _, dx, dA, dB = M.grouped_lora_grads(x, None, W, A, B, 2.0, offsets, up, dtype=torch.float64)
    assert dA[1].abs().max().item() == 0.0 and dB[1].abs().max().item() == 0.0
    xs, us = x[3:], up[3:]
    assert torch.allclose(dA[2], 2.0 * (us @ B[2]).t() @ xs, atol=1e-12)
    assert torch.allclose(dB[2], 2.0 * us.t() @ (xs @ A[2].t()), atol=1e-12)
    assert torch.allclose(dx[:3], up[:3] @ W[0] + 2.0 * (up[:3] @ B[0]) @ A[0], atol=1e-12)
