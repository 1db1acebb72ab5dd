"""CPU oracle of the NF4 weight format.  TEST INFRASTRUCTURE ONLY (see grpo_oracle.py).

The reference only switches the format on (`load_in_4bit=True`,
src/art/dev/model.py:29); the arithmetic is bitsandbytes' (not in the reference
tree, not installed here): PARITY UNPINNED against that package.  This module
restates the published scheme (Dettmers et al., "QLoRA", 2023): block-wise
absolute maximum, the 16 NormalFloat levels, two codes per byte with the first
element in the high nibble, and the optional second quantisation of the block
maxima (8-bit codes into a 256-entry code book, one fp32 scale per 256 blocks,
scalar offset).  The 8-bit code book is an input here, as it is stored with a
quantised checkpoint.  Pinned in tests/test_oracle_quant.py by a hand-packed
example, exact cases (0, +-absmax), level symmetry and the round-trip error bound.
"""
from __future__ import annotations

import numpy as np

NF4_LEVELS = np.array([
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0], dtype=np.float32)


def quantize(x: np.ndarray, blocksize: int = 64):
    """x float32 [n] (n % blocksize == 0) -> (packed uint8 [n/2], absmax float32 [n/blocksize]).
    Nearest level of x / absmax."""
    x = np.asarray(x, dtype=np.float32).reshape(-1, blocksize)
    absmax = np.abs(x).max(axis=1).astype(np.float32)
    safe = np.where(absmax == 0, np.float32(1), absmax)
    y = x / safe[:, None]
    codes = np.abs(y[..., None] - NF4_LEVELS[None, None, :]).argmin(axis=-1).astype(np.uint8).reshape(-1)
    packed = (codes[0::2] << 4) | codes[1::2]
    return packed.astype(np.uint8), absmax


def dequantize(packed: np.ndarray, absmax: np.ndarray, blocksize: int = 64) -> np.ndarray:
    """float32 [n]: level[code] * absmax[block], one fp32 multiplication."""
    codes = np.empty(packed.size * 2, dtype=np.uint8)
    codes[0::2] = packed >> 4
    codes[1::2] = packed & 15
    scale = np.repeat(np.asarray(absmax, dtype=np.float32), blocksize)
    return (NF4_LEVELS[codes] * scale).astype(np.float32)


def nested_absmax(absmax_q: np.ndarray, code2: np.ndarray, absmax2: np.ndarray, offset: float) -> np.ndarray:
    """Block maxima from their 8-bit form: code2[q] * absmax2[block // 256] + offset (fp32, two roundings)."""
    idx = np.arange(absmax_q.size) // 256
    prod = (np.asarray(code2, dtype=np.float32)[absmax_q] * np.asarray(absmax2, dtype=np.float32)[idx])
    return (prod.astype(np.float32) + np.float32(offset)).astype(np.float32)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16, as uint16 bit patterns."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r
