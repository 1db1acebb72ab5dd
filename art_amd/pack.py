"""Packer and on-disk format of the training batches.

Counterpart of src/art/local/pack.py: `packed_tensors_from_tokenized_results`
(:41-147) turns tokenized trajectories into the eight [N, S] `PackedTensors`,
`packed_tensors_to_dir` / `packed_tensors_from_dir` (:150-180) keep them as
headerless raw arrays `{key}.pt` shared between the backend and the training
process.  Same inputs, same outputs, same files; the row assignment is the
reference's sequential rule, everything per token is array work on buffers that
are written once (the reference grows eight Python lists token by token and
slices every one of them after every result).  `to_device` stages a row through
pinned memory for the kernels.
"""
from __future__ import annotations

import os
import random
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

PackedTensors = Dict[str, torch.Tensor]

# key -> dtype, the order and types of src/art/local/pack.py:158-167
DISK_DTYPES = {
    "tokens": torch.long,
    "group_ids": torch.long,
    "parent_ids": torch.long,
    "input_pos": torch.long,
    "assistant_mask": torch.bool,
    "logprobs": torch.float32,
    "advantages": torch.float32,
    "weights": torch.float32,
}


@dataclass
class TokenizedResult:
    """The fields of the reference's `TokenizedResult` (src/art/local/tokenize.py:11-22)
    that the packer reads; objects of the reference's own class work as well."""
    token_ids: Sequence[int]
    input_pos: Sequence[int]
    assistant_mask: Sequence[int]
    logprobs: Sequence[float]
    advantage: float
    prompt_id: int = 0
    prompt_length: int = 0


def packed_tensors_from_tokenized_results(tokenized_results: Sequence, seq_len: int, pad_token_id: int = -100,
                                          truncate_long_results: bool = True, verbosity: int = 1,
                                          rng=random) -> PackedTensors:
    """Same contract as the reference function.  `rng` (the `random` module by
    default, as in the reference) supplies one `randint` per packed result and the
    final `shuffle`, in the reference's order."""
    # pass 1: the sequential placement rule on lengths only
    placed = []          # (row, result index, first token taken, tokens taken, group id)
    row_len = [0]
    row_prompts = [set()]
    arrays = []
    for idx, result in enumerate(tokenized_results):
        n = len(result.token_ids)
        if n > seq_len and not truncate_long_results:
            if verbosity > 1:
                print("Result is too long, skipping")
            continue
        mask = np.asarray(result.assistant_mask, dtype=np.int64)
        pl = result.prompt_length
        n_assist_tail = int(mask[pl:].sum())
        if n_assist_tail == 0:
            if verbosity > 1:
                print("Result has no unique completion tokens, skipping")
            continue
        add = n - pl if result.prompt_id in row_prompts[-1] else n
        if row_len[-1] + add > seq_len:
            row_len.append(0)
            row_prompts.append(set())
        group_id = rng.randint(-(2 ** 63), 2 ** 63 - 1)
        start = pl if result.prompt_id in row_prompts[-1] else 0
        take = min(n - start, seq_len - row_len[-1]) if truncate_long_results else n - start
        # weight of the trajectory: the reference divides by the mask sum of what it appends
        n_assist = n_assist_tail if start else int(mask.sum())
        placed.append((len(row_len) - 1, idx, start, take, group_id, n_assist, row_len[-1]))
        # ids present in the row decide whether a later result drops its prompt
        # (the reference tests `prompt_id in group_ids[-1]`, which also holds the random ids)
        taken_prompt = max(0, min(pl - start, take))
        if taken_prompt > 0:
            row_prompts[-1].add(result.prompt_id)
        if take > taken_prompt:
            row_prompts[-1].add(group_id)
        row_len[-1] += take
        arrays.append(mask)

    n_rows = len(row_len)
    permutation = list(range(n_rows))
    rng.shuffle(permutation)
    where = [0] * n_rows                    # old row -> new row
    for new, old in enumerate(permutation):
        where[old] = new

    # pass 2: write every result once into the padded [N, S] buffers
    tokens = np.full((n_rows, seq_len), pad_token_id, dtype=np.int64)
    group_ids = np.full((n_rows, seq_len), -1, dtype=np.int64)
    parent_ids = np.full((n_rows, seq_len), -1, dtype=np.int64)
    input_pos = np.zeros((n_rows, seq_len), dtype=np.int64)
    assistant_mask = np.zeros((n_rows, seq_len), dtype=np.bool_)
    logprobs = np.full((n_rows, seq_len), np.nan, dtype=np.float32)
    advantages = np.zeros((n_rows, seq_len), dtype=np.float32)
    weights = np.zeros((n_rows, seq_len), dtype=np.float32)
    for (row, idx, start, take, group_id, n_assist, at), mask in zip(placed, arrays):
        if take <= 0:
            continue
        result = tokenized_results[idx]
        r = where[row]
        sl = slice(at, at + take)
        src = slice(start, start + take)
        tokens[r, sl] = np.asarray(result.token_ids[src], dtype=np.int64)
        input_pos[r, sl] = np.asarray(result.input_pos[src], dtype=np.int64)
        assistant_mask[r, sl] = mask[src] != 0
        logprobs[r, sl] = np.asarray(result.logprobs[src], dtype=np.float32)
        advantages[r, sl] = np.float32(result.advantage)
        weights[r, sl] = np.float32(1 / (n_assist + 1e-6))
        parent_ids[r, sl] = result.prompt_id
        n_prompt = max(0, min(result.prompt_length - start, take))
        group_ids[r, at:at + n_prompt] = result.prompt_id
        group_ids[r, at + n_prompt:at + take] = group_id

    mask_t = torch.from_numpy(assistant_mask)
    weights_t = torch.from_numpy(weights)
    weights_t = torch.where(mask_t, weights_t, torch.zeros_like(weights_t))
    weights_t[mask_t] /= weights_t[mask_t].mean()
    return {
        "tokens": torch.from_numpy(tokens),
        "group_ids": torch.from_numpy(group_ids),
        "parent_ids": torch.from_numpy(parent_ids),
        "input_pos": torch.from_numpy(input_pos),
        "assistant_mask": mask_t,
        "logprobs": torch.from_numpy(logprobs),
        "advantages": torch.from_numpy(advantages),
        "weights": weights_t,
    }


def packed_tensors_from_dir(dir: str, num_sequences: int, sequence_length: int) -> PackedTensors:
    """Shared memory maps of `{dir}/{key}.pt` (headerless raw arrays, created if missing)."""
    os.makedirs(dir, exist_ok=True)
    return {
        key: torch.from_file(f"{dir}/{key}.pt", shared=True, size=num_sequences * sequence_length,
                             dtype=dtype).view(num_sequences, sequence_length)
        for key, dtype in DISK_DTYPES.items()
    }


def packed_tensors_to_dir(tensors: PackedTensors, dir: str) -> dict:
    os.makedirs(dir, exist_ok=True)
    disk = {"dir": dir, "num_sequences": tensors["tokens"].shape[0],
            "sequence_length": tensors["tokens"].shape[1]}
    for key, tensor in packed_tensors_from_dir(**disk).items():
        tensor.copy_(tensors[key])
    return disk


class RowStager:
    """Moves packed rows to the GPU one at a time, the way the training loop consumes them
    (rows `[offset : offset + 1]`, src/art/local/service.py:96-104), with the copy of row i+1
    overlapping the step on row i.

    Two slots, each a set of pinned host buffers (allocated pinned: registering existing
    memory is not supported everywhere) and a set of device buffers.  A row goes
    file / host tensor -> pinned slot -> device slot on a copy stream of its own; the consumer's
    stream waits for one event per row, and the copy stream waits for the event the consumer's
    stream records when it is done with the slot, so nothing synchronises a whole stream or the
    device.  The host only blocks when it wants to refill a pinned slot whose previous copy
    (two rows ago) has not left yet."""

    DEPTH = 2

    def __init__(self, sequence_length: int, device: torch.device):
        self.device = torch.device(device)
        self.copy_stream = torch.cuda.Stream(self.device)  # default priority
        self.slots = []
        for _ in range(self.DEPTH):
            self.slots.append({
                "pinned": {key: torch.empty((1, sequence_length), dtype=dtype).pin_memory()
                           for key, dtype in DISK_DTYPES.items()},
                "dev": {key: torch.empty((1, sequence_length), dtype=dtype, device=self.device)
                        for key, dtype in DISK_DTYPES.items()},
                "copied": torch.cuda.Event(),     # recorded on the copy stream after the H2D copies
                "released": torch.cuda.Event(),   # recorded on the consumer's stream when it moves on
                "in_flight": False,
            })

    def _stage(self, tensors: PackedTensors, row: int, slot: dict) -> None:
        if slot["in_flight"]:
            slot["copied"].synchronize()          # the pinned buffers are about to be overwritten
        for key, buf in slot["pinned"].items():
            buf.copy_(tensors[key][row:row + 1])
        self.copy_stream.wait_event(slot["released"])   # no-op for an event never recorded
        with torch.cuda.stream(self.copy_stream):
            for key, buf in slot["pinned"].items():
                slot["dev"][key].copy_(buf, non_blocking=True)
            slot["copied"].record(self.copy_stream)
        slot["in_flight"] = True

    def rows(self, tensors: PackedTensors):
        """Yields the rows of `tensors` (host tensors or the memory maps of
        `packed_tensors_from_dir`) as dicts of device tensors [1, S].  A yielded dict stays
        valid until the generator is advanced once more (advancing hands its device buffers to
        the copy of the row after next); work on it must be enqueued, before that, on the
        stream that is current when the generator is advanced.  Closing or abandoning the
        generator early is safe: the slot of the last yielded row is released then."""
        n = tensors["tokens"].shape[0]
        if n == 0:
            return
        self._stage(tensors, 0, self.slots[0])
        pending = None   # slot of the row the consumer holds, not yet released
        try:
            for i in range(n):
                consumer = torch.cuda.current_stream(self.device)
                if pending is not None:
                    # everything the consumer enqueued for row i-1 precedes this point of its stream
                    pending["released"].record(consumer)
                    pending = None
                if i + 1 < n:
                    self._stage(tensors, i + 1, self.slots[(i + 1) % self.DEPTH])
                slot = self.slots[i % self.DEPTH]
                consumer.wait_event(slot["copied"])
                pending = slot
                yield dict(slot["dev"])
        finally:
            if pending is not None:
                pending["released"].record(torch.cuda.current_stream(self.device))

    def to_device(self, tensors: PackedTensors, row: int) -> PackedTensors:
        """One row, ready on the current stream (fresh device tensors, no overlap)."""
        slot = self.slots[0]
        self._stage(tensors, row, slot)
        consumer = torch.cuda.current_stream(self.device)
        consumer.wait_event(slot["copied"])
        out = {key: t.clone() for key, t in slot["dev"].items()}
        slot["released"].record(consumer)
        return out
