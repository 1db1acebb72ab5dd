"""Pins of the attention oracle: the visibility rule by brute force, the
attention against torch's own scaled_dot_product_attention, known structure of
a packed row."""
import math
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import attn_oracle  # noqa: E402

from art_amd import synthetic  # noqa: E402


def test_visibility_brute_force():
    g = torch.Generator().manual_seed(0)
    for _ in range(20):
        S = 17
        group = torch.randint(0, 4, (1, S), generator=g)
        parent = torch.randint(0, 4, (1, S), generator=g)
        vis = attn_oracle.visibility(group, parent)
        for i in range(S):
            for j in range(S):
                want = j <= i and (group[0, i] == group[0, j] or parent[0, i] == group[0, j])
                assert bool(vis[0, i, j]) == bool(want)


def test_bias_values():
    group = torch.tensor([[5, 5, 7, 7, -1]])
    parent = torch.tensor([[5, 5, 5, 5, -1]])
    bias = attn_oracle.attn_bias(group, parent)[0]
    inf = float("-inf")
    want = torch.tensor([[0, inf, inf, inf, inf], [0, 0, inf, inf, inf], [0, 0, 0, inf, inf],
                         [0, 0, 0, 0, inf], [inf, inf, inf, inf, 0]])
    assert torch.equal(bias, want)


def test_packed_row_structure():
    group, parent = synthetic.packed_row_ids(1, 64, 2, 4, 3, 8)
    vis = attn_oracle.visibility(group.view(1, -1), parent.view(1, -1))[0]
    # a completion token sees its prompt and the earlier tokens of its own completion only
    i = 4 + 8 + 3  # 4th token of the 2nd completion of prompt 0
    assert vis[i].nonzero().flatten().tolist() == [0, 1, 2, 3, 12, 13, 14, 15]
    # padding sees earlier padding only
    assert vis[63].nonzero().flatten().tolist() == list(range(56, 64))
    assert attn_oracle.visible_pairs(group, parent) == int(vis.sum())


def test_attention_matches_torch_sdpa():
    g = torch.Generator().manual_seed(3)
    S, Hq, Hkv, D = 48, 4, 2, 16
    q = torch.randn(S, Hq, D, generator=g)
    k = torch.randn(S, Hkv, D, generator=g)
    v = torch.randn(S, Hkv, D, generator=g)
    group, parent = synthetic.packed_row_ids(2, S, 2, 4, 2, 8)
    out, lse = attn_oracle.attention(q, k, v, group, parent, dtype=torch.float64)
    vis = attn_oracle.visibility(group.view(1, -1), parent.view(1, -1))[0]
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.double().permute(1, 0, 2), k.double().permute(1, 0, 2).repeat_interleave(2, 0),
        v.double().permute(1, 0, 2).repeat_interleave(2, 0), attn_mask=vis).permute(1, 0, 2)
    assert (out - ref).abs().max().item() < 1e-12
    # lse by explicit loop for one (head, query)
    h, i = 3, 20
    s = [(q[i, h].double() @ k[j, h // 2].double()).item() / math.sqrt(D) for j in range(S) if vis[i, j]]
    assert abs(lse[h, i].item() - math.log(sum(math.exp(x) for x in s))) < 1e-12


def test_attention_grads_finite_difference():
    g = torch.Generator().manual_seed(4)
    S, Hq, Hkv, D = 16, 2, 1, 8
    q = torch.randn(S, Hq, D, generator=g, dtype=torch.float64)
    k = torch.randn(S, Hkv, D, generator=g, dtype=torch.float64)
    v = torch.randn(S, Hkv, D, generator=g, dtype=torch.float64)
    d_out = torch.randn(S, Hq, D, generator=g, dtype=torch.float64)
    group, parent = synthetic.packed_row_ids(5, S, 1, 4, 2, 5)
    _, dq, dk, dv = attn_oracle.attention_grads(q, k, v, group, parent, d_out, dtype=torch.float64)
    f = lambda q_, k_, v_: (attn_oracle.attention(q_, k_, v_, group, parent, dtype=torch.float64)[0] * d_out).sum()
    eps = 1e-6
    for t, grad in ((q, dq), (k, dk), (v, dv)):
        for idx in ((3, 0, 2), (9, 0, 5), (15, 0, 7)):
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = [tp if x is t else x for x in (q, k, v)]
            args_m = [tm if x is t else x for x in (q, k, v)]
            fd = (f(*args_p) - f(*args_m)) / (2 * eps)
            assert abs(fd.item() - grad[idx].item()) < 1e-6


def test_attention_rows_equals_full():
    g = torch.Generator().manual_seed(6)
    S, Hq, Hkv, D = 64, 4, 2, 16
    q = torch.randn(S, Hq, D, generator=g)
    k = torch.randn(S, Hkv, D, generator=g)
    v = torch.randn(S, Hkv, D, generator=g)
    group, parent = synthetic.packed_row_ids(7, S, 2, 5, 2, 12)
    out, lse = attn_oracle.attention(q, k, v, group, parent, dtype=torch.float64)
    rows = torch.tensor([0, 4, 5, 17, 33, 58, 63])
    o2, l2 = attn_oracle.attention_rows(q, k, v, group, parent, rows, dtype=torch.float64)
    assert (o2 - out[rows]).abs().max().item() < 1e-12 and (l2 - lse[:, rows]).abs().max().item() < 1e-12
