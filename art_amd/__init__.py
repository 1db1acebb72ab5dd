"""MI355X-native GRPO training hot path (logprob/loss kernels and LoRA linear).

The compute lives in ``csrc/libartk.so`` (hand-written HIP for gfx950 behind a
C-ABI, see ``include/artk.h``).  This package is the thin host side that mirrors
the call surface of the reference's ``src/art/local/train.py``.
"""
from . import ops  # noqa: F401
from .train import (  # noqa: F401
    shift_tensor,
    _calculate_logprobs,
    calculate_logprobs,
    grpo_loss,
    fused_grpo_loss,
    get_compute_loss_fn,
)

__version__ = "0.1.0"
