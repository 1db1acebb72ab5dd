"""CPU oracle of the packer.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

Restates, list by list, what `packed_tensors_from_tokenized_results` does
(src/art/local/pack.py:41-147): results are appended to the current row while
they fit (a result whose prompt is already in the row is appended without its
prompt), otherwise a new row is opened; every completion gets a fresh random
64-bit group id; rows are shuffled; rows are padded to `seq_len`; weights are
1/(assistant tokens of the trajectory), zeroed off the mask and divided by their
mean over the mask.  The random draws follow the reference's order (one
`randint` per packed result, then one `shuffle`), so with the same seeded
generator the output is the reference's, bit for bit.  Pinned by hand-computed
cases in tests/test_oracle_pack.py; the reference's function itself cannot be
imported here (its module needs matplotlib/seaborn and the art package needs
openai, all absent).
"""
from __future__ import annotations

import random
from dataclasses import dataclass, field
from typing import List

import torch


@dataclass
class Result:
    """The fields of `TokenizedResult` (src/art/local/tokenize.py:11-22) the packer reads."""
    token_ids: List[int]
    input_pos: List[int]
    assistant_mask: List[int]
    logprobs: List[float]
    advantage: float
    prompt_id: int = 0
    prompt_length: int = 0

    def without_prompt(self) -> "Result":
        n = self.prompt_length
        return Result(self.token_ids[n:], self.input_pos[n:], self.assistant_mask[n:], self.logprobs[n:],
                      self.advantage, self.prompt_id, 0)


def pack(results: List[Result], seq_len: int, pad_token_id: int = -100, truncate_long_results: bool = True,
         rng=random):
    keys = ("token_ids", "group_ids", "parent_ids", "input_pos", "assistant_mask", "logprobs", "advantages",
            "weights")
    rows = {k: [[]] for k in keys}

    for result in results:
        if len(result.token_ids) > seq_len and not truncate_long_results:
            continue
        stripped = result.without_prompt()
        if sum(stripped.assistant_mask) == 0:
            continue
        add = len(stripped.token_ids) if result.prompt_id in rows["group_ids"][-1] else len(result.token_ids)
        if len(rows["token_ids"][-1]) + add > seq_len:
            for k in keys:
                rows[k].append([])
        group_id = rng.randint(-(2 ** 63), 2 ** 63 - 1)
        if result.prompt_id in rows["group_ids"][-1]:
            result = stripped
        n = len(result.token_ids)
        rows["token_ids"][-1].extend(result.token_ids)
        rows["group_ids"][-1].extend([result.prompt_id] * result.prompt_length
                                     + [group_id] * (n - result.prompt_length))
        rows["parent_ids"][-1].extend([result.prompt_id] * n)
        rows["input_pos"][-1].extend(result.input_pos)
        rows["assistant_mask"][-1].extend(result.assistant_mask)
        rows["logprobs"][-1].extend(result.logprobs)
        rows["advantages"][-1].extend([result.advantage] * n)
        rows["weights"][-1].extend([1 / (sum(result.assistant_mask) + 1e-6)] * n)
        if truncate_long_results:
            for k in keys:
                rows[k][-1] = rows[k][-1][:seq_len]

    permutation = list(range(len(rows["token_ids"])))
    rng.shuffle(permutation)
    for k in keys:
        rows[k] = [rows[k][i] for i in permutation]

    def pad(values, pad_value):
        for v in values:
            v.extend([pad_value] * (seq_len - len(v)))
        return values

    mask = torch.tensor(pad(rows["assistant_mask"], 0), dtype=torch.bool)
    weights = torch.tensor(pad(rows["weights"], 0.0))
    weights = torch.where(mask, weights, torch.zeros_like(weights))
    weights[mask] /= weights[mask].mean()
    return {
        "tokens": torch.tensor(pad(rows["token_ids"], pad_token_id)),
        "group_ids": torch.tensor(pad(rows["group_ids"], -1)),
        "parent_ids": torch.tensor(pad(rows["parent_ids"], -1)),
        "input_pos": torch.tensor(pad(rows["input_pos"], 0)),
        "assistant_mask": mask,
        "logprobs": torch.tensor(pad(rows["logprobs"], float("nan"))),
        "advantages": torch.tensor(pad(rows["advantages"], 0.0)),
        "weights": weights,
    }
