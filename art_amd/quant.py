"""4-bit NormalFloat base weights for the LoRA linear.

With `load_in_4bit=True` (src/art/dev/model.py:29) the reference's frozen linear
weights are stored as NF4 codes by bitsandbytes and dequantised in front of every
matmul.  `NF4Weight` holds that storage form on the GPU.  `art_amd.lora.LoRALinear`
takes it as its frozen weight (`LoRALinear.from_nf4`): the bf16 values then exist only
inside each forward / backward call, in the call's workspace, so neither a bf16 copy
nor a transposed copy stays resident (0.56 bytes per weight element instead of 4).
`dequantize()` / `dequantize_transposed()` give resident bf16 tensors for callers that
prefer to pay the memory (no dequantisation per call: about 3 % of a projection's time).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops

NF4_LEVELS = (-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
              -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
              0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
              0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0)


class NF4Weight:
    """A frozen [out, in] weight as NF4 codes + block maxima (block size 64 by default)."""

    def __init__(self, packed: torch.Tensor, shape: Tuple[int, int], absmax: Optional[torch.Tensor] = None,
                 absmax_q: Optional[torch.Tensor] = None, code2: Optional[torch.Tensor] = None,
                 absmax2: Optional[torch.Tensor] = None, offset: float = 0.0, blocksize: int = 64):
        self.packed, self.shape, self.blocksize = packed.reshape(-1), tuple(shape), blocksize
        self.absmax, self.absmax_q, self.code2, self.absmax2, self.offset = absmax, absmax_q, code2, absmax2, offset

    @classmethod
    def from_float(cls, W: torch.Tensor, blocksize: int = 64) -> "NF4Weight":
        """Quantise a device tensor (nearest level of x / block maximum)."""
        shape = tuple(W.shape)
        x = W.detach().float().reshape(-1, blocksize)
        absmax = x.abs().amax(dim=1)
        y = x / torch.where(absmax == 0, torch.ones_like(absmax), absmax).unsqueeze(1)
        levels = torch.tensor(NF4_LEVELS, dtype=torch.float32, device=W.device)
        codes = (y.unsqueeze(-1) - levels).abs().argmin(dim=-1).to(torch.uint8).reshape(-1)
        packed = (codes[0::2] << 4) | codes[1::2]
        return cls(packed.contiguous(), shape, absmax=absmax.contiguous(), blocksize=blocksize)

    def dequantize(self, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """bf16 [out, in]."""
        flat = ops.nf4_dequant(self.packed, self.absmax, self.absmax_q, self.code2, self.absmax2, self.offset,
                               self.blocksize, None if out is None else out.view(-1))
        return flat.view(self.shape)

    def dequantize_transposed(self) -> torch.Tensor:
        """bf16 [in, out], the operand of the input-gradient GEMM, written transposed straight from the codes."""
        return ops.nf4_dequant_t(self.packed, self.shape[0], self.shape[1], self.absmax, self.absmax_q,
                                 self.code2, self.absmax2, self.offset, self.blocksize)

    def nbytes(self) -> int:
        """Bytes of device memory the storage form occupies."""
        return sum(t.numel() * t.element_size() for t in
                   (self.packed, self.absmax, self.absmax_q, self.code2, self.absmax2) if t is not None)
