"""ctypes binding of the artk C-ABI (include/artk.h).

There is no fallback: if the shared library has not been built, importing the
ops fails with instructions, and every wrapper raises on a non-zero return code.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libartk.so")

ERR_INVALID_ARGUMENT = -1
ERR_WORKSPACE_TOO_SMALL = -2
ERR_UNSUPPORTED_SHAPE = -3

_i32, _i64, _sz, _f32, _p = C.c_int32, C.c_int64, C.c_size_t, C.c_float, C.c_void_p

# name -> (restype, argtypes); mirrors include/artk.h one to one.
SIGNATURES = {
    "artk_abi_version": (_i32, []),
    "artk_last_error": (C.c_char_p, []),
    "artk_logprob_fwd_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "artk_logprob_fwd": (_i32, [_p, _p, _p, _i32, _i64, _i64, _i64, _i64, _p, _p, _p, _sz, _p]),
    "artk_logprob_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "artk_logprob_bwd": (
        _i32,
        [_p, _p, _p, _p, _i32, _i64, _i64, _i64, _i64, _p, _p, _p, _i64, _p, _sz, _p],
    ),
    "artk_grpo_loss_workspace_bytes": (_sz, [_i64]),
    "artk_grpo_loss": (
        _i32,
        [_p, _p, _p, _p, _p, _p, _i32, _i64, _i64, _f32, _f32, _f32, _p, _p, _p, _sz, _p],
    ),
    "artk_grpo_loss_static": (
        _i32, [_p, _p, _p, _p, _p, _p, _i32, _i64, _i64, _f32, _f32, _f32, _p, _p, _p]),
    "artk_grpo_fused_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "artk_grpo_fused": (
        _i32,
        [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _f32, _f32, _f32, _i64, _i32, _p,
         _p, _p, _p, _sz, _p],
    ),
    "artk_transpose_bf16": (_i32, [_p, _p, _i64, _i64, _p]),
    "artk_gemm_nt": (_i32, [_p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "artk_lora_linear_fwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "artk_lora_linear_fwd": (
        _i32, [_p, _p, _p, _p, _p, _f32, _i64, _i64, _i64, _i32, _p, _p, _p, _sz, _p]),
    "artk_lora_linear_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "artk_lora_linear_bwd": (
        _i32, [_p, _p, _p, _p, _p, _p, _f32, _i64, _i64, _i64, _i32, _p, _p, _p, _p, _sz, _p]),
    "artk_moe_route_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "artk_moe_route": (_i32, [_p, _i64, _i32, _i32, _p, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "artk_moe_lora_grouped_fwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32, _i32]),
    "artk_moe_lora_grouped_fwd": (
        _i32, [_p, _p, _p, _p, _p, _f32, _p, _p, _p, _i64, _i64, _i64, _i32, _i32, _p, _p, _p, _sz, _p]),
    "artk_moe_lora_grouped_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32, _i32]),
    "artk_moe_lora_grouped_bwd": (
        _i32, [_p, _p, _p, _p, _p, _p, _p, _f32, _p, _p, _p, _i64, _i64, _i64, _i32, _i32, _p, _p, _p,
               _p, _sz, _p]),
    "artk_attn_plan_bytes": (_sz, [_i64]),
    "artk_attn_plan": (_i32, [_p, _p, _i64, _p, _sz, _p]),
    "artk_attn_fwd_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "artk_attn_fwd": (
        _i32, [_p, _p, _p, _p, _i64, _i32, _i32, _i32] + [_i64] * 8 + [_f32, _p, _p, _p, _sz, _p]),
    "artk_attn_bwd_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32]),
    "artk_attn_bwd": (
        _i32, [_p, _p, _p, _p, _p, _p, _p, _i64, _i32, _i32, _i32, C.POINTER(_i64), _f32, _p, _p, _p, _p,
               _sz, _p]),
    "artk_attn_bwd_tuning": (_i32, [_i32]),
    "artk_sumsq_f32_workspace_bytes": (_sz, []),
    "artk_sumsq_f32": (_i32, [_p, _i64, _p, _p, _sz, _p]),
    "artk_adamw_step": (_i32, [_p, _p, _p, _p, _p, _i64, _f32, _f32, _f32, _f32, _f32, _i32, _p, _f32, _p]),
    "artk_nf4_dequant": (_i32, [_p, _p, _p, _p, _p, _f32, _i64, _i32, _p, _p]),
    "artk_transpose_bf16_batched": (_i32, [_p, _p, _i64, _i64, _i64, _p]),
    "artk_profile_enable": (_i32, [_i32]),
    "artk_profile_collect": (_i32, [_i32, C.POINTER(C.c_double), C.POINTER(_i64)]),
    "artk_mfma_loop": (_i32, [_p, _i64, _i64, _i32, _p, _p]),
    "artk_mfma_loop16": (_i32, [_p, _i64, _i64, _i32, _p, _p]),
    "artk_stream_copy": (_i32, [_p, _p, _i64, _p]),
    "artk_gemm_loop_probe": (_i32, [_p, _p, _p, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _p, _p]),
    "artk_lds_probe": (_i32, [_i32, _i32, _i32, _p, _i64, _i32, _p, _p]),
}



class LoraProjStruct(C.Structure):
    """artk_lora_proj_t of include/artk.h."""
    _fields_ = [("W", _p), ("W_t", _p), ("A", _p), ("B", _p), ("bias", _p), ("y", _p), ("g", _p), ("xa", _p),
                ("dA", _p), ("dB", _p), ("out", _i64), ("r", _i32)]


class Nf4Struct(C.Structure):
    """artk_nf4_t of include/artk.h."""
    _fields_ = [("packed", _p), ("absmax", _p), ("absmax_q", _p), ("code2", _p), ("absmax2", _p),
                ("offset", _f32), ("blocksize", _i32)]


SIGNATURES.update({
    "artk_adamw8bit_step": (_i32, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _f32, _f32, _f32, _f32, _f32, _i32,
                                   _p, _f32, _p]),
    "artk_nf4_dequant_t": (_i32, [_p, _p, _p, _p, _p, _f32, _i64, _i64, _i32, _p, _p]),
    "artk_lora_linear_fwd_nf4_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "artk_lora_linear_fwd_nf4": (
        _i32, [_p, C.POINTER(Nf4Struct), _p, _p, _p, _f32, _i64, _i64, _i64, _i32, _p, _p, _p, _sz, _p]),
    "artk_lora_linear_bwd_nf4_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "artk_lora_linear_multi_fwd_workspace_bytes": (_sz, [_i64, _i64, C.POINTER(LoraProjStruct), _i32]),
    "artk_lora_linear_multi_fwd": (_i32, [_p, C.POINTER(LoraProjStruct), _i32, _f32, _i64, _i64, _p, _sz, _p]),
    "artk_lora_linear_multi_bwd_workspace_bytes": (_sz, [_i64, _i64, C.POINTER(LoraProjStruct), _i32]),
    "artk_lora_linear_multi_bwd": (_i32, [_p, C.POINTER(LoraProjStruct), _i32, _f32, _i64, _i64, _p, _p, _sz, _p]),
    "artk_lora_linear_bwd_nf4": (
        _i32, [_p, _p, C.POINTER(Nf4Struct), _p, _p, _p, _f32, _i64, _i64, _i64, _i32, _p, _p, _p, _p, _sz, _p]),
})

_lib = None


def load() -> C.CDLL:
    """Load libartk.so (built by ``__graft_entry__.build()`` / ``make -C art_amd/csrc``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built. Build it with `make -C {os.path.dirname(LIB_PATH)}` "
            "(needs hipcc; cross-compiles for gfx950 without a GPU). There is no CPU fallback."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class ArtkError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"artk error {code}: {message}")
        self.code = code


def check(code: int) -> None:
    """Raise for a non-zero return code of an artk_* call made on this thread."""
    if code == 0:
        return
    msg = load().artk_last_error().decode("utf-8", "replace")
    if code < 0:
        raise ValueError(f"artk error {code}: {msg}")
    raise ArtkError(code, msg)
