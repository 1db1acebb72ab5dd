"""Pins of the packer oracle (hand-computed rows) and bit-exact parity of the
array packer against it on random inputs, including truncation, prompt sharing,
skipped results and empty rows.  CPU only."""
import math
import os
import random
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import pack_oracle  # noqa: E402

from art_amd import pack  # noqa: E402


class FixedRng:
    """randint returns 1000, 1001, ...; shuffle keeps the order."""

    def __init__(self):
        self.next = 1000

    def randint(self, a, b):
        self.next += 1
        return self.next - 1

    def shuffle(self, x):
        pass


def R(n_prompt, n_completion, prompt_id, adv, base=0):
    n = n_prompt + n_completion
    return pack_oracle.Result(
        token_ids=list(range(base, base + n)), input_pos=list(range(n)),
        assistant_mask=[0] * n_prompt + [1] * n_completion,
        logprobs=[float("nan")] * n_prompt + [-0.5 - 0.01 * i for i in range(n_completion)],
        advantage=adv, prompt_id=prompt_id, prompt_length=n_prompt)


def test_oracle_known_rows():
    # two completions of prompt 7 (3 prompt + 2 / 3 completion tokens), then one of prompt 9 that
    # does not fit the 10-token row any more
    results = [R(3, 2, 7, 1.5, 100), R(3, 3, 7, -0.5, 200), R(2, 2, 9, 2.0, 300)]
    out = pack_oracle.pack(results, 10, pad_token_id=-100, rng=FixedRng())
    assert out["tokens"].tolist() == [[100, 101, 102, 103, 104, 203, 204, 205, -100, -100],
                                      [300, 301, 302, 303] + [-100] * 6]
    assert out["group_ids"].tolist() == [[7, 7, 7, 1000, 1000, 1001, 1001, 1001, -1, -1],
                                         [9, 9, 1002, 1002] + [-1] * 6]
    assert out["parent_ids"].tolist() == [[7] * 8 + [-1, -1], [9] * 4 + [-1] * 6]
    assert out["input_pos"].tolist() == [[0, 1, 2, 3, 4, 3, 4, 5, 0, 0], [0, 1, 2, 3, 0, 0, 0, 0, 0, 0]]
    assert out["assistant_mask"].tolist() == [[False] * 3 + [True] * 5 + [False] * 2,
                                              [False] * 2 + [True] * 2 + [False] * 6]
    assert out["advantages"][0].tolist() == [1.5] * 5 + [-0.5] * 3 + [0.0, 0.0]
    # weights: 1/2, 1/3, 1/2 per assistant token, divided by their mean over the 7 masked tokens
    raw = [1 / (2 + 1e-6)] * 2 + [1 / (3 + 1e-6)] * 3 + [1 / (2 + 1e-6)] * 2
    mean = sum(raw) / 7
    w = out["weights"]
    assert torch.allclose(w[0, 3:8], torch.tensor(raw[:5]) / mean, rtol=1e-6)
    assert w[0, :3].abs().sum().item() == 0 and w[0, 8:].abs().sum().item() == 0
    assert abs(w[out["assistant_mask"]].mean().item() - 1.0) < 1e-6
    assert math.isnan(out["logprobs"][0, 0].item()) and out["logprobs"][0, 3].item() == pytest.approx(-0.5)
    assert math.isnan(out["logprobs"][1, 9].item())


def test_oracle_truncation_and_skips():
    # a result longer than the row: the empty first row stays, the result is cut to 8 tokens
    out = pack_oracle.pack([R(2, 10, 5, 1.0)], 8, rng=FixedRng())
    assert out["tokens"].shape == (2, 8)
    assert out["tokens"][0].tolist() == [-100] * 8 and out["tokens"][1].tolist() == list(range(8))
    # not truncating: skipped, one empty row
    out = pack_oracle.pack([R(2, 10, 5, 1.0)], 8, truncate_long_results=False, rng=FixedRng())
    assert out["tokens"].shape == (1, 8) and out["assistant_mask"].sum().item() == 0
    # no completion tokens outside the prompt: skipped
    r = R(4, 0, 5, 1.0)
    out = pack_oracle.pack([r], 8, rng=FixedRng())
    assert out["tokens"].tolist() == [[-100] * 8]


def same(a, b):
    assert a.keys() == b.keys()
    for k in a:
        assert a[k].dtype == b[k].dtype and a[k].shape == b[k].shape, k
        if a[k].dtype.is_floating_point:
            assert torch.equal(torch.isnan(a[k]), torch.isnan(b[k])), k
            assert torch.equal(a[k].nan_to_num(0.0), b[k].nan_to_num(0.0)), k
        else:
            assert torch.equal(a[k], b[k]), k


@pytest.mark.parametrize("seed", range(12))
def test_packer_matches_oracle_bit_exact(seed):
    g = random.Random(seed)
    seq_len = g.choice([32, 64, 100])
    results = []
    for _ in range(g.randint(1, 40)):
        n_prompt = g.randint(0, 20)
        n_comp = g.randint(0, 50 if seed % 3 else 120)
        n = n_prompt + n_comp
        mask = [0] * n_prompt + [g.randint(0, 1) for _ in range(n_comp)]
        results.append(pack_oracle.Result(
            token_ids=[g.randint(0, 50000) for _ in range(n)], input_pos=list(range(n)), assistant_mask=mask,
            logprobs=[float("nan") if not m else -g.random() for m in mask], advantage=g.uniform(-2, 2),
            prompt_id=g.randint(0, 4), prompt_length=n_prompt))
    for truncate in (True, False):
        ref = pack_oracle.pack(results, seq_len, pad_token_id=151643, truncate_long_results=truncate,
                               rng=random.Random(seed + 100))
        got = pack.packed_tensors_from_tokenized_results(results, seq_len, pad_token_id=151643,
                                                         truncate_long_results=truncate,
                                                         rng=random.Random(seed + 100))
        same(ref, got)


def test_disk_round_trip(tmp_path):
    results = [R(3, 5, 7, 1.5, 100), R(3, 6, 7, -0.5, 200), R(2, 9, 9, 2.0, 300)]
    tensors = pack.packed_tensors_from_tokenized_results(results, 16, rng=random.Random(1))
    disk = pack.packed_tensors_to_dir(tensors, str(tmp_path / "packed"))
    assert disk["num_sequences"] == tensors["tokens"].shape[0] and disk["sequence_length"] == 16
    # headerless raw arrays with the dtypes of the reference (pack.py:158-167)
    sizes = {"tokens": 8, "group_ids": 8, "parent_ids": 8, "input_pos": 8, "assistant_mask": 1, "logprobs": 4,
             "advantages": 4, "weights": 4}
    for key, itemsize in sizes.items():
        assert os.path.getsize(tmp_path / "packed" / f"{key}.pt") == disk["num_sequences"] * 16 * itemsize
    same(tensors, pack.packed_tensors_from_dir(**disk))
